"""Row gather of the CPU restatement against NumPy's take."""
import numpy as np
import pytest

from oracle import binding as orc


@pytest.mark.parametrize("dtype,shape", [(np.float32, (128,)), (np.float32, (602,)), (np.float16, (3,)),
                                         (np.uint8, ()), (np.int64, ()), (np.float64, (2, 5)),
                                         (np.uint8, (7,))])
def test_gather_rows_is_take(dtype, shape):
    rng = np.random.default_rng(3)
    table = rng.integers(0, 200, size=(1000,) + shape).astype(dtype)
    ids = rng.integers(0, 1000, size=5000)
    out, bad = orc.gather_rows(table, ids)
    assert bad == 0 and out.dtype == table.dtype
    assert np.array_equal(out, np.take(table, ids, axis=0))


def test_ids_outside_the_table_give_zero_rows():
    table = np.arange(40, dtype=np.float32).reshape(10, 4) + 1
    ids = np.array([0, 10, 9, -1, 3, 1 << 40])
    out, bad = orc.gather_rows(table, ids)
    assert bad == 3
    assert np.array_equal(out[[0, 2, 4]], table[[0, 9, 3]])
    assert not out[[1, 3, 5]].any()


def test_empty_inputs():
    out, bad = orc.gather_rows(np.zeros((5, 3), np.float32), np.zeros(0, np.int64))
    assert out.shape == (0, 3) and bad == 0
    out, bad = orc.gather_rows(np.zeros((5, 0), np.float32), np.array([1, 2]))
    assert out.shape == (2, 0) and bad == 0
