from .block import Block, create_block_from_coo, create_block_from_csc  # noqa: F401
from .dataloader import SeedGenerator  # noqa: F401
from .synthetic import batched_seeds, chung_lu_csc, coo_to_csc, rmat_csc  # noqa: F401
from .gather import gather_pinned_tensor_rows, gather_rows  # noqa: F401
