"""The no-allocation row sum (jzhip_sum_rows_noalloc) against jzhip_sum_rows
through the C ABI: two calls in a row, the second with a smaller input, then
shapes that take each kernel form, the size limit and the allocation count.
Reductions are held to relative 1e-4; with the same chunking the two entry
points combine the same partial sums in the same order, so they also agree bit
for bit, which is asserted where the workspace and the fixed array both hold
every partial."""
import numpy as np
import pytest

from util import dev_empty, dptr, to_dev, to_host

pytestmark = pytest.mark.gpu

TOL_RED = 1e-4


def both(gpu, a, numrow, numcol, ld):
    da = to_dev(a)
    want, got = dev_empty(numrow), dev_empty(numrow)
    gpu.sum_rows(dptr(want), dptr(da), numrow, numcol, ld)
    gpu.sum_rows_noalloc(dptr(got), dptr(da), numrow, numcol, ld)
    gpu.synchronize()
    return to_host(got), to_host(want)


def check(got, want, a, numrow, numcol, ld):
    exact = a.reshape(numcol, ld)[:, :numrow].astype(np.float64).sum(axis=0)
    scale = np.abs(a.reshape(numcol, ld)[:, :numrow]).astype(np.float64).sum(axis=0) + 1e-30
    assert np.max(np.abs(got - want) / scale) <= TOL_RED
    assert np.max(np.abs(got - exact) / scale) <= TOL_RED
    assert np.array_equal(got, want)


def test_two_calls_in_a_row_second_smaller(gpu):
    r = np.random.default_rng(7)
    # first call: many column chunks, partials fill a good part of the array
    numrow, numcol = 2048, 16384
    a = r.normal(0, 1, numrow * numcol).astype(np.float32)
    got, want = both(gpu, a, numrow, numcol, numrow)
    check(got, want, a, numrow, numcol, numrow)
    # second call, smaller: must not pick up anything the first one left behind
    numrow, numcol = 512, 300
    a = r.normal(0, 1, numrow * numcol).astype(np.float32)
    got, want = both(gpu, a, numrow, numcol, numrow)
    check(got, want, a, numrow, numcol, numrow)


@pytest.mark.parametrize("numrow,numcol,pad", [(1, 1, 0), (3, 100000, 0), (64, 25088, 0), (10, 128, 0),
                                               (256, 4096, 0), (257, 1000, 3), (1000, 77, 8), (65536, 64, 0)])
def test_kernel_forms(gpu, numrow, numcol, pad):
    r = np.random.default_rng(numrow + numcol)
    ld = numrow + pad
    a = r.normal(0, 1, ld * numcol).astype(np.float32)
    got, want = both(gpu, a, numrow, numcol, ld)
    check(got, want, a, numrow, numcol, ld)


def test_rejects_sizes_beyond_the_fixed_scratch(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    numrow, numcol = 65540, 4
    da = to_dev(np.zeros(numrow * numcol, np.float32))
    out = dev_empty(numrow)
    rc = lib.jzhip_sum_rows_noalloc(dptr(out), dptr(da), numrow, numcol, numrow)
    assert rc == -3
    assert b"fixed scratch" in lib.jzhip_error_string(rc)
    assert lib.jzhip_sum_rows_noalloc(None, dptr(da), 4, 4, 4) == -1
    assert lib.jzhip_sum_rows_noalloc(dptr(out), dptr(da), 4, 4, 2) == -1


def test_creates_no_workspace(gpu):
    """The lazily created workspace is the library's only allocation: its size
    must not move across calls of the no-allocation entry point."""
    from juzhen_amd import capi
    lib = capi.load()
    before = lib.jzhip_workspace_bytes()
    r = np.random.default_rng(3)
    numrow, numcol = 512, 16384
    a = r.normal(0, 1, numrow * numcol).astype(np.float32)
    da = to_dev(a)
    out = dev_empty(numrow)
    gpu.sum_rows_noalloc(dptr(out), dptr(da), numrow, numcol, numrow)
    gpu.synchronize()
    assert lib.jzhip_workspace_bytes() == before
