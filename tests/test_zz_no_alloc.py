"""gs_csc_col_count_static (fixed scratch inside the library, no allocation)
against gs_csc_col_count (caller's workspace): identical prefix arrays, bit for
bit, on two calls in a row of which the second is smaller."""
import numpy as np
import pytest
import torch

from gsampler_amd import capi

pytestmark = pytest.mark.gpu


def _graph(num_cols, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    deg = torch.randint(0, 40, (num_cols,), generator=g, device="cuda")
    deg[::7] = 0
    indptr = torch.zeros(num_cols + 1, dtype=torch.int64, device="cuda")
    indptr[1:] = torch.cumsum(deg, 0)
    return indptr, g


def _static_count(indptr, ids, fanout, replace):
    l = capi.lib()
    n = ids.numel()
    out = torch.full((n + 1,), -7, dtype=torch.int64, device="cuda")
    capi.check(l.gs_csc_col_count_static(indptr.data_ptr(), indptr.numel() - 1,
                                         ids.data_ptr() if n else None, n, fanout,
                                         int(replace), out.data_ptr(), capi._stream()))
    return out


def test_static_count_matches_workspace_count_twice():
    indptr, g = _graph(1_000_000, 3)
    num_cols = indptr.numel() - 1
    # 10.5 M items: more than 4096 scan tiles (spine launch); then 300 K; then 5
    for n, fanout, replace in ((10_500_000, 10, False), (300_000, -1, False),
                               (5, 15, True), (0, 5, False)):
        ids = torch.randint(-3, num_cols + 3, (n,), generator=g, device="cuda")
        want = capi.col_count(indptr, ids, fanout, replace) if n else \
            torch.zeros(1, dtype=torch.int64, device="cuda")
        got = _static_count(indptr, ids, fanout, replace)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (n, fanout, replace)
        deg = torch.where((ids >= 0) & (ids < num_cols),
                          indptr[(ids.clamp(0, num_cols - 1)) + 1] - indptr[ids.clamp(0, num_cols - 1)],
                          torch.zeros_like(ids))
        cnt = deg if fanout < 0 else (torch.where(deg > 0, fanout, 0) if replace
                                      else deg.clamp(max=fanout))
        assert int(got[-1]) == int(cnt.sum())


def test_static_count_rejects_oversize():
    l = capi.lib()
    indptr, _ = _graph(1000, 4)
    rc = l.gs_csc_col_count_static(indptr.data_ptr(), 1000, indptr.data_ptr(), 1 << 27, 5, 0,
                                   indptr.data_ptr(), capi._stream())
    assert rc == 1 and b"exceed" in l.gs_last_error()
