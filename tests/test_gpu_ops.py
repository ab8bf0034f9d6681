"""Parity of every C-ABI entry point (include/nebula_hip.h) against the CPU oracle on the same
seeded inputs.  Bars: bit-exact for the im2col gather, maxpool values + argmax, avgpool, shortcut,
bias and the relu/leaky/relie activations; max|a-b| / max|ref| <= 1e-4 for conv / FC / LSTM /
softmax / batchnorm and the exp-based activations."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402

TOL = 1e-4


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


def announce(*what):
    print("CASE", *what, flush=True)


IM2COL = [(3, 9, 9, 3, 1, 1), (2, 11, 7, 5, 2, 2), (3, 35, 35, 11, 4, 0), (4, 6, 8, 1, 1, 0), (2, 8, 8, 3, 2, 1),
          (3, 14, 14, 7, 2, 3), (5, 10, 12, 3, 1, 0)]


@pytest.mark.parametrize("shape", IM2COL)
def test_im2col_gather_bit_exact(ctx, shape):
    announce("im2col", shape)
    c, h, w, k, s, p = shape
    rng = np.random.default_rng(sum(shape))
    im = rng.standard_normal((c, h, w)).astype(np.float32)
    got = ctx.im2col(ctx.array(im), k, s, p).numpy()
    want = ob.im2col(im, k, s, p)
    assert got.shape == want.shape
    np.testing.assert_array_equal(bits(got), bits(want))


CONV = [
    # B, C, H, W, F, k, s, p, bn, act
    (2, 3, 12, 12, 5, 3, 1, 1, False, "linear"),
    (3, 3, 35, 35, 16, 11, 4, 0, False, "relu"),          # AlexNet conv1 geometry
    (2, 8, 14, 14, 40, 1, 1, 0, True, "leaky"),           # 1x1
    (2, 16, 14, 14, 24, 3, 2, 1, True, "relu"),           # stride-2 3x3
    (2, 3, 30, 30, 8, 7, 2, 3, True, "relu"),             # ResNet stem geometry
    (1, 5, 9, 11, 130, 5, 1, 2, False, "logistic"),       # F > one m-tile, ragged K
    (4, 32, 7, 7, 96, 3, 1, 1, True, "linear"),
    (2, 4, 6, 6, 3, 2, 2, 1, False, "tanh"),
    # very few channels: the strip kernel's cases -- several tiles per image with a ragged last one, 2 and 3 filter
    # tiles per wave, two filter tiles per block, one channel
    (3, 3, 61, 45, 70, 7, 2, 3, True, "leaky"),
    (2, 3, 75, 75, 96, 11, 4, 0, False, "relu"),
    (2, 1, 33, 20, 150, 5, 1, 2, True, "logistic"),
    (5, 2, 16, 23, 9, 3, 1, 1, False, "linear"),
]


@pytest.mark.parametrize("case", CONV)
def test_conv_matches_oracle(ctx, case):
    from nebula_amd import hip
    announce("conv", case)
    B, Cc, H, W, F, k, s, p, bn, act = case
    rng = np.random.default_rng(abs(hash(case[:8])) % (2 ** 31))
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, Cc, k, k)) * np.sqrt(2.0 / (Cc * k * k))).astype(np.float32)
    bias = (rng.standard_normal(F) * 0.1).astype(np.float32)
    bnp = None
    if bn:
        bnp = (rng.uniform(0.8, 1.2, F).astype(np.float32), (rng.standard_normal(F) * 0.1).astype(np.float32),
               rng.uniform(0.5, 1.5, F).astype(np.float32))
    want = ob.conv_forward(x, w, bias, bnp, s, p, act)
    plan = ctx.conv_pack(w, bias, bnp, H=H, W=W, stride=s, pad=p, act=act)
    dx = ctx.array(x)
    nv = hip.lib().nbl_conv2d_num_variants()
    variants = [-1] + list(range(nv))
    if hip.lib().nbl_conv2d_plan_set_variant(plan.p, nv) == 0:      # layers with very few channels also have the strip kernel
        variants.append(nv)
    assert (nv in variants) == (Cc <= 4 and k > 1), "strip kernel eligibility changed for %r" % (case,)
    for v in variants:
        announce("conv variant", v)
        plan.set_variant(v)
        got = plan(dx).numpy()
        assert got.shape == want.shape
        assert rel(got, want) <= TOL, (case, v, rel(got, want))



SPLIT = [
    # B, C, H, W, F, k, s, p, bn, act, residual (None | "same" | "narrow"), post_act
    (4, 64, 14, 14, 64, 3, 1, 1, True, "relu", None, "linear"),
    (2, 96, 7, 7, 130, 3, 1, 1, False, "linear", "same", "relu"),       # odd plane, ragged F, fused shortcut
    (3, 128, 10, 10, 40, 1, 1, 0, True, "leaky", "narrow", "leaky"),    # 1x1 vector gather, fewer residual channels
    (1, 48, 9, 13, 24, 5, 2, 2, True, "logistic", None, "linear"),      # odd pixel count, exp-based activation
    (5, 32, 12, 12, 256, 3, 1, 1, False, "relu", "same", "linear"),     # several filter tiles per pixel tile
]


@pytest.mark.parametrize("case", SPLIT)
def test_conv_k_split_matches_oracle_and_unsplit(ctx, case):
    """A launch split along the patch rows sums in another order: within tolerance of the oracle and of the
    unsplit launch, for every tile shape, with and without the fused shortcut."""
    from nebula_amd import hip
    announce("conv split", case)
    B, Cc, H, W, F, k, s, p, bn, act, residual, post = case
    rng = np.random.default_rng(abs(hash(case[:8])) % (2 ** 31))
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, Cc, k, k)) * np.sqrt(2.0 / (Cc * k * k))).astype(np.float32)
    bias = (rng.standard_normal(F) * 0.1).astype(np.float32)
    bnp = None
    if bn:
        bnp = (rng.uniform(0.8, 1.2, F).astype(np.float32), (rng.standard_normal(F) * 0.1).astype(np.float32),
               rng.uniform(0.5, 1.5, F).astype(np.float32))
    want = ob.conv_forward(x, w, bias, bnp, s, p, act)
    OH, OW = want.shape[2:]
    conn = None
    if residual:
        conn = rng.standard_normal((B, F if residual == "same" else max(1, F // 3), OH, OW)).astype(np.float32)
        want = ob.shortcut_forward(want, conn, post)
    plan = ctx.conv_pack(w, bias, bnp, H=H, W=W, stride=s, pad=p, act=act)
    dx = ctx.array(x)
    dconn = ctx.array(conn) if conn is not None else None
    run = (lambda: plan.with_shortcut(dx, dconn, post).numpy()) if residual else (lambda: plan(dx).numpy())
    split_seen = 0
    for v in range(hip.lib().nbl_conv2d_num_variants()):
        plan.set_variant(v)
        plan.set_split(0)
        unsplit = run()
        assert plan.last_launch() == (v, 1)
        plan.set_split(1)
        announce("conv split variant", v)
        got = run()
        split_seen += plan.last_launch()[1] > 1
        assert rel(got, want) <= TOL, (case, v, rel(got, want))
        assert rel(got, unsplit) <= 1e-5, (case, v, rel(got, unsplit))
        again = run()
        np.testing.assert_array_equal(bits(got), bits(again))           # fixed summation order
    assert split_seen >= 3, "the cost model was expected to split most tile shapes of %r" % (case,)
    # a slice count chosen by hand (fewer only where the patch rows run out)
    plan.set_variant(4)
    for slices in (2, 3, 8):
        announce("conv forced slices", slices)
        plan.set_split(slices)
        got = run()
        assert 1 <= plan.last_launch()[1] <= slices
        assert rel(got, want) <= TOL, (case, slices, rel(got, want))
    plan.set_variant(-1)
    plan.set_split(-1)
    got = run()
    assert rel(got, want) <= TOL


def random_conv_case(seed):
    """A seeded geometry: channel counts either side of the tap-major rule (C % 16 == 0) and of the strip kernel
    (C <= 4), ragged filter counts, odd and even planes, every cheap activation and one exp-based, and a residual that
    has the output's shape, fewer channels, more channels, twice the size (read at stride 2), or is absent."""
    rng = np.random.default_rng(1000 + seed)
    C = int(rng.choice([1, 3, 4, 5, 8, 16, 24, 32, 48, 64]))
    k = int(rng.choice([1, 1, 2, 3, 3, 5]))
    s = int(rng.choice([1, 1, 2]))
    p = int(rng.integers(0, k // 2 + 2))
    H, W = int(rng.integers(max(k, 4), 24)), int(rng.integers(max(k, 4), 24))
    F = int(rng.choice([1, 7, 32, 40, 64, 96, 130, 200]))
    B = int(rng.integers(1, 5))
    act = str(rng.choice(["linear", "relu", "leaky", "relie", "logistic"]))
    post = str(rng.choice(["linear", "relu", "leaky"]))
    residual = str(rng.choice(["none", "same", "narrow", "wide", "double"]))
    bn = bool(rng.integers(0, 2))
    return B, C, H, W, F, k, s, p, bn, act, residual, post


@pytest.mark.parametrize("seed", range(32))
def test_conv_random_geometries_every_tile_shape(ctx, seed):
    from nebula_amd import hip
    case = random_conv_case(seed)
    announce("conv random", seed, case)
    B, Cc, H, W, F, k, s, p, bn, act, residual, post = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, Cc, k, k)) * np.sqrt(2.0 / (Cc * k * k))).astype(np.float32)
    bias = (rng.standard_normal(F) * 0.1).astype(np.float32)
    bnp = None
    if bn:
        bnp = (rng.uniform(0.8, 1.2, F).astype(np.float32), (rng.standard_normal(F) * 0.1).astype(np.float32),
               rng.uniform(0.5, 1.5, F).astype(np.float32))
    want = ob.conv_forward(x, w, bias, bnp, s, p, act)
    OH, OW = want.shape[2:]
    conn = None
    if residual != "none":
        cc = {"same": F, "narrow": max(1, F // 3), "wide": F + 5, "double": max(1, F // 2)}[residual]
        ch, cw = (2 * OH, 2 * OW) if residual == "double" else (OH, OW)
        conn = rng.standard_normal((B, cc, ch, cw)).astype(np.float32)
        want = ob.shortcut_forward(want, conn, post)
    plan = ctx.conv_pack(w, bias, bnp, H=H, W=W, stride=s, pad=p, act=act)
    dx = ctx.array(x)
    dconn = ctx.array(conn) if conn is not None else None
    run = (lambda: plan.with_shortcut(dx, dconn, post).numpy()) if conn is not None else (lambda: plan(dx).numpy())
    for v in [-1] + list(range(hip.lib().nbl_conv2d_num_variants())):
        for split in (0, 1):
            announce("conv random variant", v, "split", split)
            plan.set_variant(v)
            plan.set_split(split if v >= 0 else -1)
            got = run()
            assert got.shape == want.shape
            assert rel(got, want) <= TOL, (case, v, split, rel(got, want))
            if v < 0:
                break


def test_conv_relu_mask_matches_on_clear_margins(ctx):
    # outputs further than the tolerance from zero must land on the same side of the ReLU
    announce("conv relu mask")
    rng = np.random.default_rng(21)
    x = rng.standard_normal((2, 6, 16, 16)).astype(np.float32)
    w = (rng.standard_normal((12, 6, 3, 3)) * 0.2).astype(np.float32)
    b = (rng.standard_normal(12) * 0.1).astype(np.float32)
    pre = ob.conv_forward(x, w, b, None, 1, 1, "linear")
    want = ob.conv_forward(x, w, b, None, 1, 1, "relu")
    got = ctx.conv_pack(w, b, None, H=16, W=16, stride=1, pad=1, act="relu")(ctx.array(x)).numpy()
    clear = np.abs(pre) > 1e-4 * np.abs(pre).max()
    np.testing.assert_array_equal((got > 0)[clear], (want > 0)[clear])


@pytest.mark.parametrize("name", ob.ACT_NAMES[1:])
def test_activation_kernels(ctx, name):
    announce("activation", name)
    rng = np.random.default_rng(ob.ACT[name])
    x = np.concatenate([rng.standard_normal(70001) * 4, rng.uniform(-10, 10, 30000),
                        np.arange(-9, 9.5, 0.5), [0.0, -0.0, 1e-30, -1e-30]]).astype(np.float32)
    want = ob.activate(name, x)
    got = ctx.activation(ctx.array(x), name).numpy()
    if name in ("relu", "leaky", "relie", "linear", "hardtan", "lhtan", "plse", "ramp", "stair"):
        np.testing.assert_array_equal(bits(got), bits(want))      # no transcendental involved
    else:
        ok = np.isfinite(want)
        assert rel(got[ok], want[ok]) <= 1e-6
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    if name in ("relu", "leaky", "relie"):
        np.testing.assert_array_equal(got > 0, x > 0)               # the mask itself


IMAGES = [(2, 13, 17, 3, 13, 17), (3, 40, 30, 3, 16, 12), (2, 31, 29, 3, 47, 18), (1, 8, 8, 3, 227, 227), (2, 64, 48, 1, 5, 5),
          (1, 375, 500, 3, 224, 224), (2, 16, 20, 3, 8, 10), (1, 9, 12, 3, 18, 24), (1, 454, 454, 3, 227, 227)]


@pytest.mark.parametrize("case", IMAGES)
def test_image_to_input_bit_exact(ctx, case):
    """Device-side image preprocessing (resize, / 255, plane swap) equals the CPU restatement bit for bit."""
    announce("image_to_input", case)
    n, h, w, c, dh, dw = case
    rng = np.random.default_rng(sum(case))
    imgs = rng.integers(0, 256, (n, h, w, c), dtype=np.uint8)
    got = ctx.image_to_input(ctx.array(imgs, dtype=np.uint8), dh, dw).numpy()
    for i in range(n):
        want = ob.image_to_input(imgs[i], dh, dw)
        np.testing.assert_array_equal(bits(got[i]), bits(want))
    # same geometry again (cached tap tables), other pixels
    imgs2 = rng.integers(0, 256, (n, h, w, c), dtype=np.uint8)
    got2 = ctx.image_to_input(ctx.array(imgs2, dtype=np.uint8), dh, dw).numpy()
    np.testing.assert_array_equal(bits(got2[0]), bits(ob.image_to_input(imgs2[0], dh, dw)))


def test_copy_d2d(ctx):
    from nebula_amd import hip
    announce("copy_d2d")
    rng = np.random.default_rng(5)
    for n in (1, 3, 4, 1023, 70001):
        a = rng.standard_normal(n).astype(np.float32)
        src, dst = ctx.array(a), ctx.array(np.zeros(n, np.float32))
        ctx.copy(dst, src)
        np.testing.assert_array_equal(bits(dst.numpy()), bits(a))
    # a copy long enough for the streaming-store kernel (32 MiB and more), with a ragged tail
    n = (40 << 20) // 4 + 3
    a = rng.standard_normal(n).astype(np.float32)
    src, dst = ctx.array(a), ctx.array(np.zeros(n, np.float32))
    ctx.copy(dst, src)
    np.testing.assert_array_equal(bits(dst.numpy()), bits(a))
    big = ctx.array(np.arange(64, dtype=np.float32))
    rc = hip.lib().nbl_copy_d2d(ctx.h, big.ptr + 16, big.ptr, 64)
    assert rc == -1 and b"overlap" in hip.lib().nbl_last_error(ctx.h)


def test_activation_rejects_undefined(ctx):
    from nebula_amd import hip
    d = ctx.array(np.zeros(8, np.float32))
    for bad in (0, 14, -3):
        rc = hip.lib().nbl_activation_fwd(ctx.h, d.ptr, 8, bad)
        assert rc == -1
        assert b"undefined activation" in hip.lib().nbl_last_error(ctx.h)


POOL = [(2, 3, 12, 12, 3, 2, 1), (2, 2, 13, 11, 3, 2, 0), (1, 4, 8, 8, 2, 2, 0), (2, 5, 7, 7, 7, 7, 0),
        (1, 2, 9, 9, 2, 1, 1), (1, 1, 6, 6, 5, 3, 2), (3, 16, 55, 55, 3, 2, 0), (2, 8, 112, 112, 3, 2, 0), (2, 4, 28, 28, 2, 2, 0),
        (1, 3, 16, 12, 3, 2, 0), (2, 2, 14, 14, 7, 7, 0), (1, 2, 21, 21, 7, 2, 3),
        # rows that are not whole 16-byte pieces (AlexNet's maps): odd plane counts, padding, stride 1, a 5x5 window, a
        # non-square plane, and AlexNet's first pool at its full size
        (5, 23, 27, 27, 3, 2, 0), (16, 40, 13, 13, 3, 2, 0), (4, 24, 27, 27, 3, 2, 1), (2, 12, 55, 55, 2, 1, 1),
        (3, 24, 31, 31, 5, 3, 2), (4, 10, 45, 39, 3, 2, 0), (128, 96, 55, 55, 3, 2, 0),
        # outputs of 32 MiB and more leave through streaming stores: ResNet's pool at batch 64, a 2x2 pool of VGG-16's
        # first; a 2x2 pool whose input is longer than 256 MiB also arrives through streaming loads
        (64, 64, 112, 112, 3, 2, 0), (16, 64, 224, 224, 2, 2, 0), (22, 64, 224, 224, 2, 2, 0)]


@pytest.mark.parametrize("geom", POOL)
def test_maxpool_values_and_argmax_bit_exact(ctx, geom):
    announce("maxpool", geom)
    B, Cc, H, W, k, s, p = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    x[0, 0, :4, :4] = 0.25                      # ties: first maximum wins
    x.ravel()[::17] = np.round(x.ravel()[::17])   # more ties
    y, idx = ctx.pool(ctx.array(x), k, s, p, "max")
    wy, widx = ob.maxpool_forward(x, k, s, p)
    np.testing.assert_array_equal(bits(y.numpy()), bits(wy))
    np.testing.assert_array_equal(idx.numpy(), widx)
    y2, none = ctx.pool(ctx.array(x), k, s, p, "max", want_index=False)
    assert none is None
    np.testing.assert_array_equal(bits(y2.numpy()), bits(wy))


def test_maxpool_sentinel(ctx):
    announce("maxpool sentinel")
    x = np.full((1, 1, 4, 4), -3e8, np.float32)
    y, idx = ctx.pool(ctx.array(x), 2, 2, 0, "max")
    wy, widx = ob.maxpool_forward(x, 2, 2, 0)
    np.testing.assert_array_equal(bits(y.numpy()), bits(wy))
    np.testing.assert_array_equal(idx.numpy(), widx)


@pytest.mark.parametrize("geom", POOL)
def test_avgpool_bit_exact(ctx, geom):
    announce("avgpool", geom)
    B, Cc, H, W, k, s, p = geom
    rng = np.random.default_rng(sum(geom) + 1)
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    got = ctx.pool(ctx.array(x), k, s, p, "avg").numpy()
    want = ob.avgpool_forward(x, k, s, p)
    np.testing.assert_array_equal(bits(got), bits(want))


# window = whole plane (the pool that ends ResNet): more planes than one block stages, even and odd plane
# sizes, a plane count that leaves a ragged last block, a stride shorter than the window, and a plane too
# large for the staged kernel (general kernel)
PLANE_AVG = [(2, 130, 4, 4, 4, 4, 0), (1, 1, 3, 3, 3, 3, 0), (2, 3, 11, 11, 11, 11, 0), (1, 300, 7, 7, 7, 5, 0),
             (1, 2, 12, 12, 12, 12, 0), (4, 512, 7, 7, 7, 7, 0)]


@pytest.mark.parametrize("geom", PLANE_AVG)
def test_avgpool_whole_plane_bit_exact(ctx, geom):
    announce("avgpool whole plane", geom)
    B, Cc, H, W, k, s, p = geom
    rng = np.random.default_rng(sum(geom) + 2)
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    got = ctx.pool(ctx.array(x), k, s, p, "avg").numpy()
    want = ob.avgpool_forward(x, k, s, p)
    assert got.shape == (B, Cc, 1, 1)
    np.testing.assert_array_equal(bits(got), bits(want))
    # closed form: the mean of the plane
    np.testing.assert_allclose(got[:, :, 0, 0], x.reshape(B, Cc, -1).astype(np.float64).mean(axis=2), rtol=0, atol=2e-6)


SHORTCUT = [((2, 4, 9, 9), (2, 16, 9, 9)), ((2, 8, 10, 10), (2, 16, 5, 5)), ((1, 6, 19, 19), (1, 6, 10, 10)),
            ((2, 8, 4, 4), (2, 4, 8, 8)), ((3, 5, 7, 7), (3, 5, 7, 7)), ((2, 16, 8, 8), (2, 16, 8, 8)),
            ((2, 8, 12, 12), (2, 32, 12, 12)), ((2, 32, 12, 12), (2, 8, 12, 12)), ((2, 8, 7, 7), (2, 8, 7, 7)),
            ((2, 8, 16, 16), (2, 24, 8, 8)), ((2, 6, 24, 24), (2, 6, 8, 8)), ((2, 4, 12, 12), (2, 8, 4, 4)),
            # outputs of 32 MiB and more (streaming stores out of place, ordinary ones in place): same shape, more
            # output channels than the connection has, a ResNet stage entry (stride 2), stride 3
            ((64, 256, 28, 28), (64, 256, 28, 28)), ((32, 128, 28, 28), (32, 512, 28, 28)),
            ((32, 256, 56, 56), (32, 512, 28, 28)), ((16, 64, 84, 84), (16, 768, 28, 28)),
            # 2 x 205 MB read: streaming loads as well
            ((64, 256, 56, 56), (64, 256, 56, 56))]


@pytest.mark.parametrize("dims", SHORTCUT)
@pytest.mark.parametrize("act", ["linear", "relu", "leaky"])
def test_shortcut_bit_exact(ctx, dims, act):
    announce("shortcut", dims, act)
    conn_shape, out_shape = dims
    rng = np.random.default_rng(sum(conn_shape) + sum(out_shape))
    conn = rng.standard_normal(conn_shape).astype(np.float32)
    prev = rng.standard_normal(out_shape).astype(np.float32)
    want = ob.shortcut_forward(prev, conn, act)
    got = ctx.shortcut(ctx.array(prev), ctx.array(conn), act).numpy()
    np.testing.assert_array_equal(bits(got), bits(want))
    # in place over prev
    dprev = ctx.array(prev)
    ctx.shortcut(dprev, ctx.array(conn), act, out=dprev)
    np.testing.assert_array_equal(bits(dprev.numpy()), bits(want))


FC = [(7, 60, 11, False, "linear"), (32, 512, 1000, False, "relu"), (64, 2048, 1000, False, "linear"),
      (128, 1024, 256, True, "leaky"), (5, 33, 3, True, "logistic"), (33, 4096, 130, False, "relu"),
      (1, 256, 64, False, "tanh"),
      # small batches stream the weight matrix: ragged k tails, neuron tails, one and two batch tiles, split and unsplit
      (32, 2500, 2000, False, "relu"), (64, 25088, 96, True, "relu"), (17, 1500, 1000, False, "logistic"),
      (48, 500, 62, True, "linear"), (64, 260, 33, False, "relu"), (2, 49152, 40, False, "relu"),
      # large batches whose 64x64 tiles alone fill the chip twice over: fan-ins of two and three k-tiles (shorter than
      # the kernel's ring of four), ragged rows and neurons, and a square product
      (600, 64, 3500, False, "relu"), (520, 96, 4000, True, "leaky"), (1024, 1024, 2048, False, "linear")]


@pytest.mark.parametrize("case", FC)
def test_fc_matches_oracle(ctx, case):
    announce("fc", case)
    B, I, O, bn, act = case
    rng = np.random.default_rng(B * 7 + I + O)
    x = rng.standard_normal((B, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) * np.sqrt(2.0 / I)).astype(np.float32)
    b = (rng.standard_normal(O) * 0.1).astype(np.float32)
    bnp = None
    if bn:
        bnp = (rng.uniform(0.8, 1.2, O).astype(np.float32), (rng.standard_normal(O) * 0.1).astype(np.float32),
               rng.uniform(0.5, 1.5, O).astype(np.float32))
    want = ob.connected_forward(x, w, b, bnp, act)
    got = ctx.fc_pack(w, b, bnp, act)(ctx.array(x)).numpy()
    assert rel(got, want) <= TOL, rel(got, want)


# the weight-streaming kernel (operand-major weights, activations through LDS) on every shape limit: one and two
# batch tiles with ragged rows, neuron counts that leave part tiles and part blocks, fan-ins of a single k block,
# of part rings and part chunks, unsplit and split launches; and VGG-16's two large connected layers at batch 32
FC_STREAM = [(1, 8, 5, False, "linear"), (32, 64, 32, False, "relu"), (31, 72, 257, True, "leaky"), (33, 264, 100, False, "relu"),
             (64, 2056, 513, True, "linear"), (17, 4096, 1000, False, "logistic"), (48, 520, 62, True, "linear"),
             (5, 12288, 2500, False, "relu"), (32, 25088, 4096, False, "relu"), (32, 4096, 4096, True, "relu"),
             (64, 9216, 4096, False, "relu")]


@pytest.mark.parametrize("case", FC_STREAM)
def test_fc_weight_streaming_kernel_matches_oracle_and_the_tiled_kernels(ctx, case):
    announce("fc stream", case)
    B, I, O, bn, act = case
    rng = np.random.default_rng(B * 11 + I + O)
    x = rng.standard_normal((B, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) * np.sqrt(2.0 / I)).astype(np.float32)
    b = (rng.standard_normal(O) * 0.1).astype(np.float32)
    bnp = None
    if bn:
        bnp = (rng.uniform(0.8, 1.2, O).astype(np.float32), (rng.standard_normal(O) * 0.1).astype(np.float32),
               rng.uniform(0.5, 1.5, O).astype(np.float32))
    ob.use_openblas(threads=8)
    want = ob.connected_forward(x, w, b, bnp, act)
    ob.use_custom_gemm()
    plan = ctx.fc_pack(w, b, bnp, act)
    dx = ctx.array(x)
    plan.set_kernel(2)
    y = ctx.empty((B, O))
    from nebula_amd import hip
    ctx.check(hip.lib().nbl_lds_fill(ctx.h, 0xffffffff))     # stale LDS must not show
    got = plan(dx, out=y).numpy()
    assert np.isfinite(got).all()
    assert rel(got, want) <= TOL, rel(got, want)
    again = plan(dx).numpy()
    np.testing.assert_array_equal(bits(again), bits(got))          # fixed summation order
    plan.set_kernel(1)
    tiled = plan(dx).numpy()
    assert rel(got, tiled) <= 2e-5, rel(got, tiled)


def test_bias_and_batchnorm_primitives(ctx):
    announce("bias/bn primitives")
    rng = np.random.default_rng(31)
    B, Cc, S = 3, 10, 77
    y = rng.standard_normal((B, Cc, S)).astype(np.float32)
    bias = rng.standard_normal(Cc).astype(np.float32)
    mean = (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    var = rng.uniform(0.01, 2, Cc).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, Cc).astype(np.float32)
    a = y.copy()
    ob.oracle().orc_forward_bias(ob._fp(a), ob._fp(bias), Cc, S, B)
    got = ctx.forward_bias(ctx.array(y), ctx.array(bias), Cc, S, B).numpy()
    np.testing.assert_array_equal(bits(got), bits(a))
    a = y.copy()
    ob.oracle().orc_batchnorm_normalize(ob._fp(a), ob._fp(mean), ob._fp(var), Cc, S, B)
    ob.oracle().orc_batchnorm_scale_down(ob._fp(a), ob._fp(scale), Cc, S, B)
    got = ctx.batchnorm_inference(ctx.array(y), ctx.array(mean), ctx.array(var), ctx.array(scale), Cc, S, B).numpy()
    assert rel(got, a) <= 1e-6


# row lengths either side of every kernel choice (4, 8 or 16 entries per thread in registers, then the general kernel)
@pytest.mark.parametrize("shape", [(6, 333), (64, 1000), (3, 10000), (1, 5), (128, 1000), (2, 1024), (2, 1025), (3, 2048),
                                   (2, 2049), (2, 8713), (2, 16384), (2, 16385), (3, 20000), (5, 1),
                                   (1024, 10000)])      # 39 MiB: leaves through streaming stores
def test_softmax(ctx, shape):
    announce("softmax", shape)
    rng = np.random.default_rng(shape[1])
    x = (rng.standard_normal(shape) * 5).astype(np.float32)
    want = ob.softmax_forward(x)
    got = ctx.softmax(ctx.array(x)).numpy()
    assert rel(got, want) <= TOL
    np.testing.assert_array_equal(got.argmax(1), want.argmax(1))
    assert np.abs(got.sum(1) - 1).max() < 1e-5
    # closed form in double, and shift invariance (the row maximum is subtracted first)
    e = np.exp(x.astype(np.float64) - x.astype(np.float64).max(1, keepdims=True))
    assert np.abs(got - e / e.sum(1, keepdims=True)).max() <= 2e-6
    shifted = ctx.softmax(ctx.array(x + np.float32(8.0))).numpy()
    assert np.abs(shifted - got).max() <= 2e-6


LSTM = [(3, 2, 5, 4, False, "linear"), (4, 3, 6, 5, True, "tanh"), (6, 8, 64, 96, False, "linear"),
        (5, 64, 128, 128, True, "linear"), (3, 70, 40, 33, False, "linear"),
        # hidden sizes that are multiples of 128 take the one-launch-per-step kernel: ragged batch tiles,
        # a non-linear sub-layer activation, odd and even numbers of load batches per wave
        (4, 37, 96, 256, False, "tanh"), (3, 33, 64, 384, True, "linear"), (2, 5, 48, 512, False, "linear")]


@pytest.mark.parametrize("case", LSTM)
def test_lstm_matches_oracle(ctx, case):
    announce("lstm", case)
    T, B, I, H, bn, act = case
    rng = np.random.default_rng(T * 100 + B + I + H)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    names = ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU")
    wt = [(rng.uniform(-1, 1, (H, H if n[1] == "W" else I)) / np.sqrt(H)).astype(np.float32) for n in names]
    bs = [(rng.uniform(-1, 1, H) / np.sqrt(H)).astype(np.float32) for n in names]
    bnp = None
    if bn:
        bnp = ([rng.uniform(0.8, 1.2, H).astype(np.float32) for _ in names],
               [(rng.standard_normal(H) * 0.1).astype(np.float32) for _ in names],
               [rng.uniform(0.5, 1.5, H).astype(np.float32) for _ in names])
    want, wcell = ob.lstm_forward(x, wt, bs, bnp, act, want_cell=True)
    plan = ctx.lstm_pack(wt, bs, bnp, act)
    cell = ctx.empty((B, H))
    got = plan(ctx.array(x), cell=cell).numpy()
    assert rel(got, want) <= TOL, rel(got, want)
    assert rel(cell.numpy(), wcell[-1]) <= TOL
    # a second call starts again from zero state
    got2 = plan(ctx.array(x)).numpy()
    np.testing.assert_array_equal(bits(got2), bits(got))


# (T1, T2, B, I, H): hidden sizes of the one-launch-per-step kernel with odd and even pass lengths (its two state
# buffers swap roles after an odd pass), of the split-K path and of the single fused kernel
LSTM_CARRY = [(3, 4, 5, 48, 256), (2, 2, 37, 64, 128), (1, 1, 33, 32, 384), (3, 2, 6, 64, 96), (2, 3, 7, 20, 33)]


@pytest.mark.parametrize("case", LSTM_CARRY)
def test_lstm_state_kept_between_passes(ctx, case):
    """lstm_layer_t never clears hidden_state / cell_state between forward() calls (lstm_layer.cu:15-140).  A carrying
    plan run on the two parts of a sequence must give what one pass over the whole sequence gives (and what the oracle
    gives for the whole sequence); reset_state and a different batch size start from zero; set_state on a second
    plan continues from y[T1-1] and the cell state the first pass returned."""
    announce("lstm carry", case)
    T1, T2, B, I, H = case
    T = T1 + T2
    rng = np.random.default_rng(T * 100 + B + I + H)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    names = ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU")
    wt = [(rng.uniform(-1, 1, (H, H if n[1] == "W" else I)) / np.sqrt(H)).astype(np.float32) for n in names]
    bs = [(rng.uniform(-1, 1, H) / np.sqrt(H)).astype(np.float32) for n in names]
    want, wcell = ob.lstm_forward(x, wt, bs, None, "linear", want_cell=True)
    plan = ctx.lstm_pack(wt, bs, None, "linear")
    whole = plan(ctx.array(x)).numpy()
    assert rel(whole, want) <= TOL
    plan.carry_state(True)
    cell1, cell2 = ctx.empty((B, H)), ctx.empty((B, H))
    first = plan(ctx.array(x[:T1]), cell=cell1).numpy()
    second = plan(ctx.array(x[T1:]), cell=cell2).numpy()
    assert rel(first, whole[:T1]) <= 1e-5 and rel(second, whole[T1:]) <= 1e-5, (rel(first, whole[:T1]), rel(second, whole[T1:]))
    assert rel(second, want[T1:]) <= TOL and rel(cell2.numpy(), wcell[-1]) <= TOL
    # a third pass goes on from the second: the same as the oracle run on the sequence with its first part repeated
    third = plan(ctx.array(x[:T1])).numpy()
    want3 = ob.lstm_forward(np.concatenate([x, x[:T1]]), wt, bs, None, "linear")
    assert rel(third, want3[T:]) <= TOL
    # a new stream, a pass of another batch size, and carrying switched off all start from zero
    plan.reset_state()
    np.testing.assert_array_equal(bits(plan(ctx.array(x[:T1])).numpy()), bits(first))
    if B > 1:
        fewer = plan(ctx.array(np.ascontiguousarray(x[:T1, :B - 1]))).numpy()
        assert rel(fewer, want[:T1, :B - 1]) <= TOL
        again = plan(ctx.array(x[:T1])).numpy()                      # the kept state belongs to B - 1 rows: not used
        np.testing.assert_array_equal(bits(again), bits(first))
    plan.carry_state(False)
    np.testing.assert_array_equal(bits(plan(ctx.array(x[:T1])).numpy()), bits(first))
    np.testing.assert_array_equal(bits(plan(ctx.array(x[:T1])).numpy()), bits(first))
    # the state handed over explicitly to another plan of the same weights
    other = ctx.lstm_pack(wt, bs, None, "linear")
    with pytest.raises(Exception):
        other.set_state(ctx.array(first[-1]), cell1)          # not carrying: refused
    other.carry_state(True)
    other.set_state(ctx.array(first[-1]), cell1)
    np.testing.assert_array_equal(bits(other(ctx.array(x[T1:])).numpy()), bits(second))


@pytest.mark.parametrize("H", [128, 33])
def test_lstm_token_input_equals_one_hot_input(ctx, H):
    """One-hot input rows given as token indices: the gather must reproduce the dense product bit for bit."""
    announce("lstm tokens", H)
    T, B, V = 5, 7, 50
    rng = np.random.default_rng(H)
    tokens = rng.integers(0, V, (T, B)).astype(np.uint32)
    tokens[2, 3] = V + 5                                  # outside the vocabulary: an all-zero input row
    x = np.zeros((T, B, V), np.float32)
    for t in range(T):
        for b in range(B):
            if tokens[t, b] < V:
                x[t, b, tokens[t, b]] = 1.0
    names = ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU")
    wt = [(rng.uniform(-1, 1, (H, H if n[1] == "W" else V)) / np.sqrt(H)).astype(np.float32) for n in names]
    bs = [(rng.uniform(-1, 1, H) / np.sqrt(H)).astype(np.float32) for n in names]
    want = ob.lstm_forward(x, wt, bs, None, "linear")
    plan = ctx.lstm_pack(wt, bs, None, "linear")
    dense = plan(ctx.array(x)).numpy()
    got = plan.from_tokens(ctx.array(tokens, dtype=np.uint32)).numpy()
    np.testing.assert_array_equal(bits(got), bits(dense))
    assert rel(got, want) <= TOL


def test_target_prob_sum_and_perplexity(ctx):
    announce("target prob sum")
    rng = np.random.default_rng(77)
    for rows, n in ((1, 5), (37, 11), (4096, 1000)):
        p = rng.random((rows, n), dtype=np.float32)
        p /= p.sum(1, keepdims=True)
        t = rng.integers(0, n, rows).astype(np.uint32)
        want = ob.target_prob_sum(p, t)
        got = ctx.target_prob_sum(ctx.array(p), ctx.array(t, dtype=np.uint32))
        assert abs(got - want) <= 1e-5 * abs(want), (rows, n, got, want)
        assert abs(got - float(p[np.arange(rows), t].astype(np.float64).sum())) <= 1e-5 * abs(want)


RNN = [(3, 2, 5, 4, False, "linear"), (4, 3, 9, 7, True, "leaky"), (5, 37, 48, 128, False, "relu"),
       (4, 64, 96, 256, True, "linear"), (1, 5, 16, 128, False, "tanh"), (3, 32, 200, 384, True, "relu")]


@pytest.mark.parametrize("case", RNN)
def test_rnn_matches_oracle(ctx, case):
    """rnn_layer_t::forward, incl. its step-0 wiring; widths that are multiples of 128 take the fused step kernel."""
    announce("rnn", case)
    T, B, I, O, bn, act = case
    rng = np.random.default_rng(T * 1000 + B + I + O)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    fan = (I, O, O)
    wt = [(rng.standard_normal((O, f)) * np.sqrt(1.0 / f)).astype(np.float32) for f in fan]
    bs = [(rng.standard_normal(O) * 0.1).astype(np.float32) for _ in fan]
    bnp = None
    if bn:
        bnp = ([rng.uniform(0.8, 1.2, O).astype(np.float32) for _ in fan],
               [(rng.standard_normal(O) * 0.1).astype(np.float32) for _ in fan],
               [rng.uniform(0.5, 1.5, O).astype(np.float32) for _ in fan])
    want = ob.rnn_forward(x, wt, bs, bnp, act)
    plan = ctx.rnn_pack(wt, bs, bnp, act)
    got = plan(ctx.array(x)).numpy()
    assert rel(got, want) <= TOL, rel(got, want)
    for t in range(T):                      # every step on its own scale (step 0 is wired differently)
        assert rel(got[t], want[t]) <= TOL, (t, rel(got[t], want[t]))
    np.testing.assert_array_equal(bits(plan(ctx.array(x)).numpy()), bits(got))


def test_topk_matches(ctx):
    announce("topk")
    rng = np.random.default_rng(41)
    for rows, n, k in ((1, 5, 1), (37, 11, 3), (128, 1000, 5), (9, 70, 70)):
        p = rng.random((rows, n), dtype=np.float32)
        p[::3, : n // 2] = p[::3, n // 2: 2 * (n // 2)]          # ties, also at the k-th place
        labels = rng.integers(0, n, rows).astype(np.uint32)
        want = ob.topk_matches(p, labels, k)
        got = ctx.topk_matches(ctx.array(p), ctx.array(labels, dtype=np.uint32), k)
        assert got == want, (rows, n, k, got, want)
        order = np.argsort(-p.astype(np.float64), axis=1, kind="stable")
        assert want == int(sum(labels[r] in order[r, :k] for r in range(rows)))


def test_error_paths(ctx):
    from nebula_amd import hip
    import ctypes as C
    l = hip.lib()
    announce("error paths")
    p = C.c_void_p()
    w = np.zeros((2, 2, 3, 3), np.float32)
    b = np.zeros(2, np.float32)
    f = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))
    assert l.nbl_conv2d_pack(ctx.h, f(w), f(b), None, None, None, 2, 8, 8, 2, 3, 1, 1, 0, C.byref(p)) == -1   # act 0
    assert l.nbl_conv2d_pack(ctx.h, f(w), f(b), None, None, None, 2, 8, 8, 2, 3, 0, 1, 11, C.byref(p)) == -1  # stride 0
    assert l.nbl_conv2d_pack(ctx.h, None, f(b), None, None, None, 2, 8, 8, 2, 3, 1, 1, 11, C.byref(p)) == -1  # NULL w
    assert l.nbl_conv2d_pack(ctx.h, f(w), f(b), f(b), None, None, 2, 8, 8, 2, 3, 1, 1, 11, C.byref(p)) == -1  # half a BN
    assert l.nbl_conv2d_pack(ctx.h, f(w), f(b), None, None, None, 2, 1, 1, 2, 3, 1, 0, 11, C.byref(p)) == -1  # k > input
    assert l.nbl_pool_fwd(ctx.h, None, None, None, 1, 1, 4, 4, 2, 2, 0, 0) == -1
    d = ctx.empty((16,))
    assert l.nbl_pool_fwd(ctx.h, d.ptr, d.ptr, None, 1, 1, 4, 4, 2, 2, 0, 7) == -1                             # mode
    # zero batch is a no-op, not an error
    plan = ctx.conv_pack(w, b, None, H=8, W=8, stride=1, pad=1, act="relu")
    assert l.nbl_conv2d_fwd(ctx.h, plan.p, d.ptr, d.ptr, 0) == 0
    # a convolution reads whole neighbourhoods while other blocks write: output and input must not share memory, and the
    # residual of a fused shortcut may be the output only as a whole
    big = ctx.empty((4 * 2 * 8 * 8,))
    assert l.nbl_conv2d_fwd(ctx.h, plan.p, big.ptr, big.ptr, 1) == -1 and b"overlap" in l.nbl_last_error(ctx.h)
    assert l.nbl_conv2d_fwd(ctx.h, plan.p, big.ptr, big.ptr + 64, 1) == -1 and b"overlap" in l.nbl_last_error(ctx.h)
    assert l.nbl_conv2d_fwd(ctx.h, plan.p, big.ptr, big.ptr + 4 * 2 * 8 * 8, 1) == 0                     # side by side is fine
    y1 = ctx.empty((4 * 2 * 8 * 8,))
    assert l.nbl_conv2d_shortcut_fwd(ctx.h, plan.p, big.ptr, y1.ptr, 2, 8, 8, y1.ptr + 16, 1, hip.ACT["relu"]) == -1
    assert b"alias" in l.nbl_last_error(ctx.h)
    assert l.nbl_conv2d_shortcut_fwd(ctx.h, plan.p, big.ptr, y1.ptr, 2, 8, 8, big.ptr, 1, hip.ACT["relu"]) == -1
    assert b"overlap" in l.nbl_last_error(ctx.h)
    assert l.nbl_conv2d_shortcut_fwd(ctx.h, plan.p, big.ptr, y1.ptr, 2, 8, 8, y1.ptr, 1, hip.ACT["relu"]) == 0   # in place
    # k-split modes: -1 (measured), 0, 1 and a slice count of 2..8
    assert l.nbl_conv2d_plan_set_split(plan.p, 9) != 0 and l.nbl_conv2d_plan_set_split(plan.p, -2) != 0
    assert l.nbl_conv2d_plan_set_split(plan.p, 8) == 0 and l.nbl_conv2d_plan_set_split(plan.p, -1) == 0
    assert l.nbl_ctx_create(99, C.byref(p)) != 0
    assert b"device" in l.nbl_last_error(None)
