"""fc_conv_implicit_gemm_static (split-reduction workspace in a static device array, no allocation)
against fc_conv_implicit_gemm with a workspace of the caller's: same bits, on two calls in a row,
the second with a smaller input; and against the fp64 oracle.  The call leaves the arena and the
device's free memory as they were, and can be recorded into a graph."""
import ctypes

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL_IM2COL = 1e-5


def cshape(s):
    import fastconv_amd as F
    return F.ConvShape(*[getattr(s, n) for n, _ in F.ConvShape._fields_])


def _free_device_bytes():
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _both(L, shp, seed):
    s = O.shape(*shp)
    cs = cshape(s)
    plan = L.igemm_plan(cs, 3)      # the 64x64 tile: small layers split their reduction over workgroups and need the workspace
    x, w = O.make_inputs(s, seed=seed)
    bias = O.rng_uniform(seed + 50, (s.K,))
    mark = L.mark()
    try:
        dx, dw, db = L.upload(x), L.upload(w), L.upload(bias)
        Wp, tab = L.alloc(plan.Wp_bytes), L.alloc(plan.table_bytes)
        nout = s.N * s.K * plan.OH * plan.OW
        y1, y2 = L.alloc(4 * nout), L.alloc(4 * nout)
        ws = L.alloc(plan.ws_bytes) if plan.ws_bytes else None
        L.igemm_pack_filter(plan, dw, Wp, tab)
        L.fill_zero(y1, 4 * nout)
        L.fill_zero(y2, 4 * nout)
        L.conv_implicit_gemm(plan, dx, Wp, tab, y1, db, True, ws)
        L.sync()
        pool_before, free_before = L.pool_stats(), _free_device_bytes()
        L.conv_implicit_gemm_static(plan, dx, Wp, tab, y2, db, True)
        L.sync()
        assert L.pool_stats() == pool_before             # nothing taken from the arena
        assert _free_device_bytes() == free_before       # nor from the device
        shape_out = (s.N, s.K, plan.OH, plan.OW)
        a, b = L.download(y1, shape_out), L.download(y2, shape_out)
    finally:
        L.release(mark)
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    return plan, a, b, truth


def test_static_workspace_entry_point_matches_the_caller_workspace_one():
    import fastconv_amd as F
    from fastconv_amd import capi
    L = F.load(0, 2 << 30)
    try:
        # a split reduction that nearly fills the static workspace, then a smaller one, then an unsplit layer
        for shp, seed in [((1, 256, 56, 56, 256, 3, 3, 1, 1, 1), 1), ((1, 512, 14, 14, 512, 3, 3, 2, 2, 1), 2),
                          ((1, 2048, 7, 7, 512, 1, 1, 1, 1, 0), 3), ((32, 64, 28, 28, 128, 3, 3, 1, 1, 1), 4)]:
            print("static workspace", shp, flush=True)
            plan, a, b, truth = _both(L, shp, seed)
            if seed < 4:
                assert plan.split_k > 1 and 0 < plan.ws_bytes <= capi.IGEMM_STATIC_WS_BYTES
            else:
                assert plan.split_k == 1
            assert np.abs(a).max() > 0
            assert np.array_equal(a, b), shp
            assert O.max_rel_err(b, truth) <= TOL_IM2COL
        # a layer whose partial sums do not fit is refused, and nothing is launched
        big = cshape(O.shape(1, 256, 56, 56, 256))
        plan = L.igemm_plan(big, 0)            # 128x128 tiles: few workgroups, many parts
        assert plan.ws_bytes > capi.IGEMM_STATIC_WS_BYTES
        buf = L.alloc(1 << 20)
        with pytest.raises(F.FastConvError) as e:
            L.conv_implicit_gemm_static(plan, buf, buf, buf, buf)
        assert e.value.status == -6 and "static" in str(e.value)
        # errors of the shared launch code name the entry point that was called
        ok = L.igemm_plan(cshape(O.shape(1, 16, 8, 8, 16)), 3)
        with pytest.raises(F.FastConvError) as e:
            L.conv_implicit_gemm_static(ok, None, buf, buf, buf)
        assert "fc_conv_implicit_gemm_static:" in str(e.value)
        # a second context on the same GPU is refused while this one owns the array, and served once it is gone
        other = F.load(0, 64 << 20)
        try:
            obuf = other.alloc(1 << 20)
            with pytest.raises(F.FastConvError) as e:
                other.conv_implicit_gemm_static(ok, obuf, obuf, obuf, obuf)
            assert e.value.status == -5 and "another context" in str(e.value)
            L.close()
            L = None
            ow, ox = other.alloc(1 << 20), other.alloc(1 << 20)
            other.fill_zero(ow, 1 << 20)
            other.fill_zero(ox, 1 << 20)
            oWp, otab, oy = other.alloc(ok.Wp_bytes), other.alloc(ok.table_bytes), other.alloc(1 << 20)
            other.igemm_pack_filter(ok, ow, oWp, otab)
            other.conv_implicit_gemm_static(ok, ox, oWp, otab, oy)
            assert not other.download(oy, (1, 16, 8, 8)).any()
        finally:
            other.close()
    finally:
        if L is not None:
            L.close()


def test_static_workspace_entry_point_inside_a_recorded_graph():
    """The use the entry point is for: a split-reduction layer recorded between fc_graph_begin and
    fc_graph_end.  Every replay, with a fresh input and eager work in between, gives the bits of the
    eager call on the same input."""
    import fastconv_amd as F
    L = F.load(0, 1 << 30)
    try:
        s = O.shape(1, 512, 14, 14, 512, 3, 3, 2, 2, 1)
        cs = cshape(s)
        plan = L.igemm_plan(cs, 3)
        assert plan.split_k > 1
        _, w = O.make_inputs(s, seed=7)
        dw = L.upload(w)
        Wp, tab = L.alloc(plan.Wp_bytes), L.alloc(plan.table_bytes)
        ws = L.alloc(plan.ws_bytes)
        nin, nout = s.N * s.C * s.H * s.W, s.N * s.K * plan.OH * plan.OW
        dx, y, yref = L.alloc(4 * nin), L.alloc(4 * nout), L.alloc(4 * nout)
        L.igemm_pack_filter(plan, dw, Wp, tab)
        L.upload_into(dx, O.rng_uniform(1, (s.N, s.C, s.H, s.W)))
        L.conv_implicit_gemm_static(plan, dx, Wp, tab, y, None, True)
        L.sync()
        L.graph_begin()
        L.conv_implicit_gemm_static(plan, dx, Wp, tab, y, None, True)
        g = L.graph_end()
        try:
            for seed in (2, 3, 4):
                print("static workspace under a graph, replay with seed", seed, flush=True)
                L.upload_into(dx, O.rng_uniform(seed, (s.N, s.C, s.H, s.W)))
                L.conv_implicit_gemm(plan, dx, Wp, tab, yref, None, True, ws)      # eager, caller's workspace
                L.fill_zero(y, 4 * nout)
                L.sync()
                L.graph_launch(g)
                a, b = L.download(yref, (s.N, s.K, plan.OH, plan.OW)), L.download(y, (s.N, s.K, plan.OH, plan.OW))
                assert np.abs(a).max() > 0
                assert np.array_equal(a, b), seed
        finally:
            L.graph_destroy(g)
    finally:
        L.close()
