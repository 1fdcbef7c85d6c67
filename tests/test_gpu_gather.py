"""Row gather through the C ABI and through the registered operator, against
the CPU restatement: every vector width the kernel picks (16, 8, 4, 2, 1 bytes),
rows shorter and longer than a wavefront's reach, tables in pinned host memory,
ids outside the table."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd import capi
from oracle import binding as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CASES = [(torch.float32, (128,)), (torch.float32, (602,)), (torch.float32, (100,)),
         (torch.float32, (1,)), (torch.float32, (3,)), (torch.float16, (3,)),
         (torch.float16, (256,)), (torch.uint8, ()), (torch.uint8, (7,)), (torch.int64, ()),
         (torch.float64, (2, 5)), (torch.float32, (4096,)), (torch.bfloat16, (129,))]


def make(dtype, shape, rows, seed):
    g = torch.Generator().manual_seed(seed)
    raw = torch.randint(0, 250, (rows,) + shape, generator=g)
    return raw.to(dtype)


def as_numpy(t):
    t = t.cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy()
    return t.numpy()


@pytest.mark.parametrize("dtype,shape", CASES)
def test_gather_rows_parity(dtype, shape):
    table = make(dtype, shape, 3000, 1)
    ids = torch.randint(0, 3000, (20011,), generator=torch.Generator().manual_seed(2))
    want, _ = orc.gather_rows(as_numpy(table), ids.numpy())
    got = capi.gather_rows(table.to(DEV), ids.to(DEV))
    assert got.shape == (ids.numel(),) + shape and got.dtype == dtype
    assert np.array_equal(as_numpy(got), want)
    op = gs.utils.gather_rows(table.to(DEV), ids.to(DEV))
    assert torch.equal(op, got)


def test_unaligned_views_fall_back_to_narrower_vectors():
    base = make(torch.float32, (130,), 500, 3).to(DEV)
    table = base[:, 1:129]            # contiguous() makes a fresh, aligned copy
    ids = torch.randint(0, 500, (999,), device=DEV)
    assert torch.equal(capi.gather_rows(table, ids), table[ids])
    flat = make(torch.uint8, (), 4099, 4).to(DEV)[3:]   # storage offset 3: 1-byte vectors
    ids = torch.randint(0, 4096, (5000,), device=DEV)
    assert torch.equal(capi.gather_rows(flat, ids), flat[ids])


def test_table_in_pinned_host_memory():
    table = make(torch.float32, (64,), 20000, 5).pin_memory()
    ids = torch.randint(0, 20000, (50000,), device=DEV)
    got = gs.utils.gather_pinned_tensor_rows(table, ids)
    assert got.is_cuda and torch.equal(got.cpu(), table[ids.cpu()])
    labels = make(torch.int64, (), 20000, 6).pin_memory()
    assert torch.equal(gs.utils.gather_rows(labels, ids).cpu(), labels[ids.cpu()])
    with pytest.raises(ValueError):
        gs.utils.gather_pinned_tensor_rows(table.to(DEV), ids)
    with pytest.raises(RuntimeError):
        gs.utils.gather_rows(make(torch.float32, (4,), 10, 7), ids)   # pageable host memory


def test_ids_outside_the_table_and_empty_inputs():
    table = make(torch.float32, (5,), 10, 8).to(DEV) + 1
    ids = torch.tensor([0, 10, 9, -1, 3, 1 << 40], device=DEV)
    got, bad = capi.gather_rows(table, ids, count_bad=True)
    assert bad == 3
    assert torch.equal(got[[0, 2, 4]], table[[0, 9, 3]]) and not got[[1, 3, 5]].any()
    got, bad = capi.gather_rows(table, ids[:0], count_bad=True)
    assert got.shape == (0, 5) and bad == 0
    assert capi.gather_rows(table[:, :0], ids[:1]).shape == (1, 0)
