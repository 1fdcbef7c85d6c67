from .matrix import Matrix  # noqa: F401
from .batch_matrix import BatchMatrix  # noqa: F401
