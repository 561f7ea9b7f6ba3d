"""The step operator entry point that allocates nothing (bnnhmc_mcmc_step_static) against the one that
takes a caller-owned workspace: same kernels, same launch, so the outputs must agree bit for bit.  Two
calls in a row on the library's static scratch, the second on a smaller input, so that whatever the
first call left in the scratch is in the way of the second."""
import sys

import numpy as np
import pytest

from hipmem import DevBuf, free_bytes, synchronize

pytestmark = pytest.mark.gpu

P = 961


def _case(pkg, lib, orc, n, L, eps, G, seed, static):
    model = lib.default_model(n=n)
    launch = lib.default_launch(cus_per_chain=G)
    X, y, th = orc.gen_window(seed, 0, n, teacher_scale=0.3, noise_sigma=5.0)
    rng = np.random.default_rng(seed)
    w0 = (th * 0.8).astype(np.float32)
    m0 = rng.normal(0, 1, P).astype(np.float32)
    g0 = orc.eval_f32(lib_om(n), X, y, w0)[2]
    dev = DevBuf.from_numpy
    dX, dy, dw0, dm0, dg0 = dev(X), dev(y), dev(w0), dev(m0), dev(g0)
    outs = [DevBuf.full(P, np.nan) for _ in range(4)]
    dloss = DevBuf.full(n + P, np.nan)
    if static:
        lib.mcmc_step_static(model, launch, dX.ptr, dy.ptr, dw0.ptr, outs[0].ptr, dm0.ptr, outs[1].ptr, dg0.ptr,
                             outs[2].ptr, outs[3].ptr, dloss.ptr, eps, L, 0)
        lib.step_check(model, launch, 0, 0)
        # The first call for a configuration has looked up the device, the launch plan and the scratch's
        # address; a second call only launches kernels: the free device memory is the same before and after
        synchronize()
        before = free_bytes()
        lib.mcmc_step_static(model, launch, dX.ptr, dy.ptr, dw0.ptr, outs[0].ptr, dm0.ptr, outs[1].ptr, dg0.ptr,
                             outs[2].ptr, outs[3].ptr, dloss.ptr, eps, L, 0)
        lib.step_check(model, launch, 0, 0)
        assert free_bytes() == before, "bnnhmc_mcmc_step_static changed the free device memory"
    else:
        wsb = lib.step_workspace_bytes(model, launch)
        ws = DevBuf.full(wsb // 4 + 16, 0, np.int32)
        lib.mcmc_step(model, launch, dX.ptr, dy.ptr, dw0.ptr, outs[0].ptr, dm0.ptr, outs[1].ptr, dg0.ptr,
                      outs[2].ptr, outs[3].ptr, dloss.ptr, ws.ptr, wsb, eps, L, 0)
        lib.step_check(model, launch, ws.ptr, 0)
    res = [o.numpy(P) for o in outs] + [dloss.numpy(n + P)]
    ref = orc.mcmc_step(lib_om(n), X, y, w0, m0, g0, eps, L)
    return res, ref


def lib_om(n):
    import orc_binding as ob

    return ob.Model(22, 40, n, ob.LIK_STUDENT_T, 100.0, 2.2, 200.0)


def test_static_scratch_step_operator_equals_the_workspace_one(pkg, lib, orc):
    # first call: one chain on 256 workgroups (the whole scratch in use); second: a smaller input on 8
    for (n, L, eps, G, seed) in [(20000, 12, 0.01, 256, 31), (1500, 7, 0.01, 8, 32)]:
        print("static step operator n=%d L=%d G=%d" % (n, L, G), flush=True)
        sys.stdout.flush()
        got, ref = _case(pkg, lib, orc, n, L, eps, G, seed, static=True)
        want, _ = _case(pkg, lib, orc, n, L, eps, G, seed, static=False)
        for a, b, name in zip(got, want, ("w_next", "mom_next", "grad_cur", "grad_next", "loss_values")):
            assert a.tobytes() == b.tobytes(), name
        assert np.all(got[3] == 0)
        # and both are the oracle's step to the tolerance of the operator's own parity test
        gscale = float(np.abs(ref[2]).max())
        assert float(np.abs(got[2] - ref[2]).max()) <= 1e-5 * max(1, L // 4) * gscale
        np.testing.assert_allclose(got[0], ref[0], rtol=0, atol=1e-6 * L * max(1.0, float(np.abs(ref[0]).max())))


def test_static_scratch_refuses_what_does_not_fit(pkg, lib):
    # 64 -> 128 -> 1 on 128 workgroups would need 8.7 MB of exchange scratch: refused before any launch
    model = lib.default_model(d0=64, d1=128, n=4096)
    launch = lib.default_launch(cus_per_chain=128)
    with pytest.raises(pkg.BnnHmcError) as e:
        lib.mcmc_step_static(model, launch, 256, 256, 256, 256, 256, 256, 256, 256, 256, 256, 0.01, 1, 0)
    assert e.value.code == pkg.ERR_INVALID and "exchange scratch" in str(e.value)
