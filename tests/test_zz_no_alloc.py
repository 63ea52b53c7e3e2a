"""The allocation-free entry point kai_matmul_noalloc against kai_matmul: same kernels, partial sums of a
reduction cut into parts in a fixed array inside the library instead of the heap scratch.  Two calls in a row,
the second with a smaller input (the array keeps the first call's contents), products that need no scratch at
all, and a product whose partial sums exceed the array (refused with a clear error)."""
import numpy as np
import pytest

from util import REL_FRO_TOL, ko, rel_fro

pytestmark = pytest.mark.gpu


def test_noalloc_matmul_matches_matmul_on_two_calls_in_a_row():
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import DeviceBuffer as DB, KaiError, VMath
    kai.load()
    kai.set_device(0)
    limit = kai.load().kai_matmul_noalloc_scratch_bytes()
    assert limit == 32 << 20
    rng = np.random.default_rng(77)

    def both(ndat, yvec, xvec, acc):
        plan = VMath.gemm_plan(0, 1, ndat, yvec, xvec)
        x = rng.standard_normal((ndat, xvec)).astype(np.float32)
        w = rng.uniform(-0.05, 0.05, (yvec, xvec)).astype(np.float32)
        y0 = rng.standard_normal((ndat, yvec)).astype(np.float32)
        dx, dw = DB.from_numpy(x), DB.from_numpy(w)
        want, got = DB.from_numpy(y0), DB.from_numpy(y0)
        VMath.matmul(0, want, dw, dx, yvec, ndat, xvec, acc)
        VMath.matmul_noalloc(0, got, dw, dx, yvec, ndat, xvec, acc)
        want, got = want.to_numpy((ndat, yvec)), got.to_numpy((ndat, yvec))
        what = "%dx%dx%d acc=%s (%s)" % (ndat, yvec, xvec, acc, plan)
        assert np.isfinite(got).all(), what
        assert rel_fro(got, want) <= REL_FRO_TOL, what
        # same plan, same kernels, sums in a fixed order: the two entry points agree bit for bit
        np.testing.assert_array_equal(got, want, err_msg=what)
        # and both agree with the oracle on a sample of rows
        rows = np.unique(rng.integers(0, ndat, 6))
        ref = ko.matmul_rows(w, x, rows)
        if acc:
            ref = ref + y0[rows]
        assert rel_fro(got[rows], ref) <= REL_FRO_TOL, what
        return plan

    # two calls in a row through the array, the second smaller: 16 parts of 256 x 512, then 16 parts of 64 x 64
    p1 = both(256, 512, 4096, False)
    p2 = both(64, 64, 4096, True)
    assert int(p1.rsplit(" ", 1)[1]) > 1 and int(p2.rsplit(" ", 1)[1]) > 1, (p1, p2)
    both(96, 4096, 4096, False)        # the 32 x 128 tile with parts
    both(100, 300, 5000, True)         # ragged tiles, parts with a shorter last one
    # products that need no scratch: one launch of the small-product kernel, the skinny stream, a large tile
    both(64, 512, 784, False)
    both(4, 4096, 4096, True)
    both(1, 4096, 4096, False)
    both(512, 2048, 1024, False)
    # a product whose partial sums do not fit the array is refused, with both sizes in the message
    ndat = yvec = 1536
    xvec = 8192
    plan = VMath.gemm_plan(0, 1, ndat, yvec, xvec)
    split = int(plan.rsplit(" ", 1)[1])
    assert split * ndat * yvec * 4 > limit, plan
    dummy = DB(ndat * xvec * 4)
    out = DB(ndat * yvec * 4)
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(0, out, dummy, dummy, yvec, ndat, xvec, False)
    assert e.value.code == 510 and str(limit) in e.value.message and str(split * ndat * yvec * 4) in e.value.message
    # the refused call left the library usable, and argument checks are those of kai_matmul
    both(64, 64, 4096, False)
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(-1, out, dummy, dummy, 4, 4, 4, False)
    assert e.value.code == 510
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(0, None, dummy, dummy, 4, 4, 4, False)
    assert e.value.code == 523
    VMath.matmul_noalloc(0, out, dummy, dummy, 0, 4, 4, False)     # empty: nothing to do
    kai.synchronize()
