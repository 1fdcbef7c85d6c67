import torch


def gather_rows(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """table[ids] along the first axis on the GPU of `ids`, for a table on that
    GPU or in pinned host memory (read in place, no staging copy): the feature /
    label fetch that follows sampling in a training loop
    (examples/graphsage/graphsage_e2e.py:113-118 of the reference)."""
    return torch.ops.gs_ops._CAPI_GatherRows(table, ids)


def gather_pinned_tensor_rows(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """Same contract as dgl.utils.gather_pinned_tensor_rows, which the reference
    imports for pinned edge data and features (python/gs/matrix_api/matrix.py:5,
    19-23)."""
    if not table.is_pinned():
        raise ValueError("gather_pinned_tensor_rows: the table is not in pinned memory")
    return gather_rows(table, ids)
