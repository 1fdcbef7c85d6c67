from .synthetic import batched_seeds, chung_lu_csc, coo_to_csc, rmat_csc  # noqa: F401
