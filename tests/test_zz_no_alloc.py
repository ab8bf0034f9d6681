"""nbl_fc_fwd_noalloc (static device scratch, no allocation) against nbl_fc_fwd and the CPU oracle.

Same kernels and the same split of the fan-in, so the two entry points must agree bit for bit; the
oracle bar is the connected layer's (max|a-b| / max|ref| <= 1e-4).  Two calls in a row share the
scratch array, the second with a smaller input, so stale partial sums of the first call would show."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402

TOL = 1e-4


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


def test_fc_noalloc_matches_fc_fwd_and_oracle_on_two_calls_in_a_row():
    from nebula_amd import hip
    ob.use_openblas(threads=8)
    rng = np.random.default_rng(77)
    I, O = 4096, 1000                       # split along the fan-in at both batch sizes
    w = (rng.standard_normal((O, I)) * np.sqrt(2.0 / I)).astype(np.float32)
    b = (rng.standard_normal(O) * 0.1).astype(np.float32)
    bn = (rng.uniform(0.8, 1.2, O).astype(np.float32), (rng.standard_normal(O) * 0.1).astype(np.float32),
          rng.uniform(0.5, 1.5, O).astype(np.float32))
    with hip.Ctx(0) as ctx:
        plan = ctx.fc_pack(w, b, bn, "leaky")
        small = ctx.fc_pack(w[:40, :96].copy(), b[:40], None, "relu")     # too few k-tiles to split: no scratch at all
        for B in (64, 17):                  # the second call is the smaller one
            print("CASE fc_noalloc batch", B, flush=True)
            x = rng.standard_normal((B, I)).astype(np.float32)
            dx = ctx.array(x)
            want = ob.connected_forward(x, w, b, bn, "leaky")
            ref = plan(dx).numpy()
            out = ctx.empty((B, O))
            ctx.check(hip.lib().nbl_fill_zero(ctx.h, out.ptr, out.nbytes))
            got = plan.noalloc(dx, out).numpy()
            np.testing.assert_array_equal(bits(got), bits(ref))
            assert rel(got, want) <= TOL, rel(got, want)
            xs = np.ascontiguousarray(x[:, :96])
            got_s = small.noalloc(ctx.array(xs), ctx.empty((B, 40))).numpy()
            np.testing.assert_array_equal(bits(got_s), bits(small(ctx.array(xs)).numpy()))
            assert rel(got_s, ob.connected_forward(xs, w[:40, :96].copy(), b[:40], None, "relu")) <= TOL


def test_fc_noalloc_refuses_what_the_scratch_cannot_hold():
    from nebula_amd import hip
    rng = np.random.default_rng(78)
    B, I, O = 1280, 4096, 2048              # 160 tiles, cut in three on a 256-CU part: 3 x 1280 x 2048 floats of partial sums
    w = (rng.standard_normal((O, I)) * 0.02).astype(np.float32)
    b = np.zeros(O, np.float32)
    with hip.Ctx(0) as ctx:
        plan = ctx.fc_pack(w, b, None, "linear")
        x = ctx.array(rng.standard_normal((B, I)).astype(np.float32))
        out = ctx.empty((B, O))
        rc = hip.lib().nbl_fc_fwd_noalloc(ctx.h, plan.p, x.ptr, out.ptr, B)
        msg = hip.lib().nbl_last_error(ctx.h).decode()
        assert rc == -4 and "static scratch" in msg, (rc, msg)          # NBL_EUNSUPPORTED
        # the allocating entry point takes the same call
        ref = plan(x).numpy()
        assert np.isfinite(ref).all()


def test_fc_noalloc_inside_a_stream_capture_replays_bit_equal():
    """The entry point is for callers that cannot allocate, a stream capture among them: captured into a HIP graph on
    the context's own stream (nothing in the call may synchronise, allocate or look a symbol up), then replayed several
    times with eager work of the same context between the replays; every replay must give nbl_fc_fwd's bits."""
    import ctypes as C
    from nebula_amd import hip
    rt = C.CDLL("libamdhip64.so")
    rng = np.random.default_rng(79)
    I, O, B = 4096, 1000, 48
    w = (rng.standard_normal((O, I)) * np.sqrt(2.0 / I)).astype(np.float32)
    b = (rng.standard_normal(O) * 0.1).astype(np.float32)
    with hip.Ctx(0) as ctx:
        plan = ctx.fc_pack(w, b, None, "relu")
        xs = [rng.standard_normal((B, I)).astype(np.float32) for _ in range(3)]
        dx = ctx.array(xs[0])
        want = [plan(ctx.array(x)).numpy() for x in xs]
        out = ctx.empty((B, O))
        stream = C.c_void_p(hip.lib().nbl_ctx_stream(ctx.h))
        ctx.sync()
        graph, graph_exec = C.c_void_p(), C.c_void_p()
        assert rt.hipStreamBeginCapture(stream, C.c_int(1)) == 0          # hipStreamCaptureModeThreadLocal
        rc = hip.lib().nbl_fc_fwd_noalloc(ctx.h, plan.p, dx.ptr, out.ptr, B)
        end = rt.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0, hip.lib().nbl_last_error(ctx.h)
        assert end == 0 and graph.value
        assert rt.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, C.c_size_t(0)) == 0
        try:
            for n, which in enumerate((0, 1, 2, 1)):
                print("CASE fc_noalloc graph replay", n, flush=True)
                dx.upload(xs[which])                                      # eager work of the program between replays
                ctx.check(hip.lib().nbl_fill_zero(ctx.h, out.ptr, out.nbytes))
                assert rt.hipGraphLaunch(graph_exec, stream) == 0
                ctx.sync()
                np.testing.assert_array_equal(bits(out.numpy()), bits(want[which]))
        finally:
            rt.hipGraphExecDestroy(graph_exec)
            rt.hipGraphDestroy(graph)
