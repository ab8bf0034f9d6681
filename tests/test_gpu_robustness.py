"""Things a kernel must not depend on, and bounds that were only stated: LDS contents left by an earlier kernel,
pointers of alias layers behind a shortcut that writes in place, and how many bits the single-precision batchnorm and
softmax kernels may differ from the CPU forms (common/batchnorm.cc:58-97, models/layers/softmax_layer.cc:85-106)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402

ob.use_openblas(threads=8)


@pytest.fixture(scope="module")
def ctx():
    from nebula_amd import hip
    c = hip.Ctx(0)
    yield c
    c.close()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


def ulps(a, b):
    """Distance in representable floats between two float32 arrays of equal sign pattern (finite values)."""
    ia = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    ib = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia)
    ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return np.abs(ia - ib)


# layers the strip kernel takes (at most 4 input channels), with patch-row counts that leave padding rows in the last
# step of 8: 3*11*11 = 363, 3*7*7 = 147, 3*3*3 = 27, 1*5*5 = 25, 4*3*3 = 36
STRIP = [(3, 227, 96, 11, 4, 0), (3, 224, 64, 7, 2, 3), (3, 64, 64, 3, 1, 1), (1, 40, 48, 5, 1, 2), (4, 33, 32, 3, 2, 1)]


@pytest.mark.parametrize("geom", STRIP)
@pytest.mark.parametrize("pattern", [0xffffffff, 0x7fc00000, 0x7f800000])
def test_strip_kernel_does_not_read_lds_it_has_not_written(ctx, geom, pattern):
    """LDS keeps what the previous kernel left.  Every CU's LDS is filled with a NaN (or Inf) bit pattern right before
    the launch: a patch row that read a word the block had not staged would turn a whole pixel into NaN."""
    from nebula_amd import hip
    C_, H, F, k, s, p = geom
    print("CASE strip kernel behind an LDS fill of 0x%08x" % pattern, geom, flush=True)
    rng = np.random.default_rng(C_ * 1000 + H)
    B = 3
    w = (rng.standard_normal((F, C_, k, k)) * np.sqrt(2.0 / (C_ * k * k))).astype(np.float32)
    b = (rng.standard_normal(F) * 0.1).astype(np.float32)
    x = rng.standard_normal((B, C_, H, H)).astype(np.float32)
    want = ob.conv_forward(x, w, b, None, s, p, "leaky")
    plan = ctx.conv_pack(w, b, None, H=H, W=H, stride=s, pad=p, act="leaky")
    plan.set_variant(hip.lib().nbl_conv2d_num_variants())          # the strip kernel
    dx = ctx.array(x)
    clean = plan(dx).numpy()
    ctx.check(hip.lib().nbl_lds_fill(ctx.h, pattern))
    y = plan(dx)
    got = y.numpy()
    assert np.isfinite(got).all()
    np.testing.assert_array_equal(bits(got), bits(clean))
    assert rel(got, want) <= 1e-4


def test_tiled_convolution_and_recurrent_steps_behind_an_lds_fill(ctx):
    from nebula_amd import hip
    print("CASE igemm tiles and lstm step behind an LDS fill", flush=True)
    rng = np.random.default_rng(77)
    B, C_, H, F = 5, 20, 13, 70                    # ragged in every direction: padded patch rows, part tiles
    w = (rng.standard_normal((F, C_, 3, 3)) * 0.1).astype(np.float32)
    b = (rng.standard_normal(F) * 0.1).astype(np.float32)
    x = rng.standard_normal((B, C_, H, H)).astype(np.float32)
    want = ob.conv_forward(x, w, b, None, 1, 1, "relu")
    plan = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="relu")
    dx = ctx.array(x)
    for v in range(hip.lib().nbl_conv2d_num_variants()):
        plan.set_variant(v)
        plan.set_split(0)
        ctx.check(hip.lib().nbl_lds_fill(ctx.h, 0xffffffff))
        got = plan(dx).numpy()
        assert np.isfinite(got).all() and rel(got, want) <= 1e-4, v
    T, Bs, I, Hd = 3, 5, 64, 128
    ws = [rng.uniform(-1, 1, (Hd, Hd if s < 4 else I)).astype(np.float32) / np.float32(np.sqrt(Hd)) for s in range(8)]
    bs = [rng.uniform(-1, 1, Hd).astype(np.float32) / np.float32(np.sqrt(Hd)) for _ in range(8)]
    xs = rng.standard_normal((T, Bs, I)).astype(np.float32)
    ob.use_custom_gemm()
    want = ob.lstm_forward(xs, ws, bs, None, "linear")
    ob.use_openblas(threads=8)
    lp = ctx.lstm_pack(ws, bs, None, "linear")
    ctx.check(hip.lib().nbl_lds_fill(ctx.h, 0xffffffff))
    got = lp(ctx.array(xs)).numpy()
    assert np.isfinite(got).all() and rel(got, want) <= 1e-4


def _block_cfg(in_place, tail):
    return ("[net]\nbatch=3\nheight=12\nwidth=12\nchannels=8\nfuse_shortcut=1\nconv_split=0\n%s"
            "[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=relu\n"
            "[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=relu\n"
            "[convolutional]\nfilters=16\nsize=1\nstride=1\npadding=0\nactivation=linear\n"
            "[shortcut]\nhops=3\nactivation=relu\n%s"
            "[connected]\noutput=24\nactivation=leaky\n"
            "[connected]\noutput=10\nactivation=linear\n[softmax]\ngroups=1\n"
            % ("shortcut_in_place=1\n" if in_place else "", tail))


@pytest.mark.parametrize("tail", ["[dropout]\nprobability=0.5\n", "[cost]\ntype=l2\n", "[dropout]\nprobability=0.5\n[dropout]\nprobability=0.1\n"])
def test_alias_layers_behind_an_in_place_shortcut_follow_the_tensor(tail):
    """A dropout or cost layer has no tensor of its own: it points at its producer's.  When the shortcut in front of it
    gives up its tensor to write over its connection's, the alias must follow, or the next layer reads freed memory.
    (A connected layer follows the alias, as in the reference's cfgs: its dropout layer reports a 1x1x1 shape.)"""
    from nebula_amd.net import Network
    print("CASE in-place shortcut followed by", tail.split("]")[0][1:], flush=True)
    rng = np.random.default_rng(3)
    outs = {}
    for in_place in (False, True):
        with Network(_block_cfg(in_place, tail)) as net:
            if not outs:
                blob = np.concatenate([(rng.standard_normal(c) * (np.sqrt(2.0 / f) if kind == "weight" else 0.1)).astype(np.float32)
                                       for _, kind, c, f in net.weight_layout()])
                x = rng.standard_normal(net.batch_size * net.input_size).astype(np.float32)
                onet = ob.OracleNet(_block_cfg(False, tail).replace("fuse_shortcut=1\n", "").replace("conv_split=0\n", ""))
                onet.load_weights(blob)
                want = onet.forward(x.reshape(3, 8, 12, 12))
            net.load_weight_blob(blob)
            net.set_input(x)
            n_alias = tail.count("[")
            shortcut = 3
            assert net.output_writer(shortcut + n_alias) == shortcut           # the alias reports the shortcut's values
            for _ in range(2):
                net.forward()
                net.sync()
            outs[in_place] = [net.output(i) for i in range(shortcut, net.num_layers)]
    for i, (a, b) in enumerate(zip(outs[False], outs[True])):
        np.testing.assert_array_equal(bits(a), bits(b), err_msg="layer %d" % (3 + i))
    assert rel(outs[True][-1], want[-1].ravel()) <= 1e-4
    assert rel(outs[True][1], want[4].ravel()) <= 1e-4          # the alias layer's own output, read back through its pointer


def test_batchnorm_kernel_differs_from_the_cpu_division_in_almost_no_element(ctx):
    """The kernel multiplies by a double-precision reciprocal where batchnorm.cc:70 divides; rounded to float the two
    differ in about one element in 2^29.  Held here on 2^24 elements: at most two differ, by one ulp."""
    print("CASE batchnorm bits", flush=True)
    rng = np.random.default_rng(41)
    B, Cc, S = 16, 64, 16384
    y = (rng.standard_normal((B, Cc, S)) * 3).astype(np.float32)
    mean = (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    var = rng.uniform(0.01, 2, Cc).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, Cc).astype(np.float32)
    a = y.copy()
    ob.oracle().orc_batchnorm_normalize(ob._fp(a), ob._fp(mean), ob._fp(var), Cc, S, B)
    ob.oracle().orc_batchnorm_scale_down(ob._fp(a), ob._fp(scale), Cc, S, B)
    got = ctx.batchnorm_inference(ctx.array(y), ctx.array(mean), ctx.array(var), ctx.array(scale), Cc, S, B).numpy()
    d = ulps(got, a)
    assert int((d != 0).sum()) <= 2 and int(d.max()) <= 1, (int((d != 0).sum()), int(d.max()))


@pytest.mark.parametrize("shape", [(512, 1000), (64, 10000), (16, 20000)])
def test_softmax_kernel_within_a_few_ulps_of_the_exact_value(ctx, shape):
    """expf, a tree-shaped float row sum and one division: every probability within 8 ulps of the exactly rounded
    value (float64 closed form of exp(x - max) / sum), on rows of every kernel variant.  The CPU form (softmax_layer.cc:85-106) adds the row
    sequentially in float, which alone moves it up to n/2 ulps from the exact value; the kernel must be no further from
    the CPU form than that bound allows."""
    print("CASE softmax bits", shape, flush=True)
    rng = np.random.default_rng(shape[1])
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    want = ob.softmax_forward(x)
    got = ctx.softmax(ctx.array(x)).numpy()
    # (the argument of the exponential is the float difference x - max in both forms: its rounding is part of the function)
    e = np.exp((x - x.max(1, keepdims=True)).astype(np.float64))
    exact = (e / e.sum(1, keepdims=True)).astype(np.float32)
    big = exact > 1e-30             # below that an ulp is a denormal step and means nothing
    assert int(ulps(got[big], exact[big]).max()) <= 8, int(ulps(got[big], exact[big]).max())      # (5 seen)
    assert int(ulps(got[big], want[big]).max()) <= 8 + shape[1] // 2
