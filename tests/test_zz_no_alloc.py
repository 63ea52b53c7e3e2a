"""The allocation-free entry point kai_matmul_noalloc against kai_matmul: same kernels, partial sums of a
reduction cut into parts in a fixed array inside the library instead of the heap scratch.

Phase 1 runs with the library's heap scratch released (kai_shutdown) and BEFORE any kai_matmul: every product is
issued through kai_matmul_noalloc only, and afterwards the heap scratch must still not exist (size, growth count and
kept bytes all 0) -- a fall-back to the heap scratch on any path would show there.  Phase 2 computes the same
products with kai_matmul and compares.  Two calls in a row, the second with a smaller input (the array keeps the
first call's contents), products that need no scratch at all, and a product whose partial sums at kai_matmul's
part count exceed the array: the entry point cuts it into fewer parts that fit instead of refusing it."""
import numpy as np
import pytest

from util import REL_FRO_TOL, ko, rel_fro

pytestmark = pytest.mark.gpu


def test_noalloc_matmul_matches_matmul_on_two_calls_in_a_row():
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import DeviceBuffer as DB, KaiError, VMath
    kai.load()
    kai.set_device(0)
    kai.synchronize()
    kai.shutdown()                      # the heap scratch is gone; nothing below may bring it back before phase 2
    assert kai.scratch_info() == (0, 0, 0)
    limit = kai.load().kai_matmul_noalloc_scratch_bytes()    # also looks up the array's address on this device
    assert limit == 32 << 20
    rng = np.random.default_rng(77)

    cases = [
        # two calls in a row through the array, the second smaller: 16 parts of 256 x 512, then 16 parts of 64 x 64
        (256, 512, 4096, False),
        (64, 64, 4096, True),
        (96, 4096, 4096, False),        # the 32 x 128 tile with parts
        (100, 300, 5000, True),         # ragged tiles, parts with a shorter last one
        # products that need no scratch: one launch of the small-product kernel, the skinny stream, a large tile
        (64, 512, 784, False),
        (4, 4096, 4096, True),
        (1, 4096, 4096, False),
        (512, 2048, 1024, False),
        # kai_matmul cuts this one into parts whose sums need more than the array: fewer parts here
        (1536, 1536, 8192, False),
        (64, 64, 4096, False),
    ]
    held = []
    for ndat, yvec, xvec, acc in cases:
        x = rng.standard_normal((ndat, xvec)).astype(np.float32)
        w = rng.uniform(-0.05, 0.05, (yvec, xvec)).astype(np.float32)
        y0 = rng.standard_normal((ndat, yvec)).astype(np.float32)
        dx, dw, got = DB.from_numpy(x), DB.from_numpy(w), DB.from_numpy(y0)
        VMath.matmul_noalloc(0, got, dw, dx, yvec, ndat, xvec, acc)
        held.append((x, w, y0, dx, dw, got.to_numpy((ndat, yvec))))
    kai.synchronize()
    assert kai.scratch_info() == (0, 0, 0), "kai_matmul_noalloc touched the heap scratch"

    # phase 2: the same products through kai_matmul (which allocates its scratch now)
    n_split = 0
    for (ndat, yvec, xvec, acc), (x, w, y0, dx, dw, got) in zip(cases, held):
        plan = VMath.gemm_plan(0, 1, ndat, yvec, xvec)
        what = "%dx%dx%d acc=%s (%s)" % (ndat, yvec, xvec, acc, plan)
        want = DB.from_numpy(y0)
        VMath.matmul(0, want, dw, dx, yvec, ndat, xvec, acc)
        want = want.to_numpy((ndat, yvec))
        assert np.isfinite(got).all(), what
        assert rel_fro(got, want) <= REL_FRO_TOL, what
        split = int(plan.rsplit(" ", 1)[1]) if " split " in plan else 1
        n_split += split > 1
        if split * ndat * yvec * 4 <= limit:
            # same plan, same kernels, sums in a fixed order: the two entry points agree bit for bit
            np.testing.assert_array_equal(got, want, err_msg=what)
        else:
            assert (ndat, yvec, xvec) == (1536, 1536, 8192), what    # the one case meant to differ in its part count
        # and both agree with the oracle on a sample of rows
        rows = np.unique(rng.integers(0, ndat, 6))
        ref = ko.matmul_rows(w, x, rows)
        if acc:
            ref = ref + y0[rows]
        assert rel_fro(got[rows], ref) <= REL_FRO_TOL, what
    assert n_split >= 5, "the cases were meant to cut their reductions into parts"
    assert kai.scratch_info()[0] > 0     # kai_matmul did allocate: the check after phase 1 was not vacuous

    # argument checks are those of kai_matmul; a dimension beyond 2^31 - 1 is refused with a message
    dummy = DB(64)
    out = DB(64)
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(-1, out, dummy, dummy, 4, 4, 4, False)
    assert e.value.code == 510
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(0, None, dummy, dummy, 4, 4, 4, False)
    assert e.value.code == 523
    with pytest.raises(KaiError) as e:
        VMath.matmul_noalloc(0, out, dummy, dummy, 1 << 31, 4, 4, False)
    assert e.value.code == 510 and "dimension" in e.value.message
    VMath.matmul_noalloc(0, out, dummy, dummy, 0, 4, 4, False)     # empty: nothing to do
    kai.synchronize()
