"""Pins for the CPU oracle that do not involve the reference at all: closed forms, brute force,
and library routines (torch on CPU).  Each one is chosen so that a plausible slip -- a transposed
operand, a wrong tap order, eps inside the root, a swapped gate -- fails it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import binding as ob


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(np.abs(b).max(), 1e-30))


def test_im2col_closed_form_bruteforce():
    rng = np.random.default_rng(0)
    for (c, h, w, k, s, p) in [(2, 6, 7, 3, 1, 1), (3, 9, 9, 5, 2, 2), (1, 11, 11, 11, 4, 0), (2, 5, 5, 2, 2, 1)]:
        im = rng.standard_normal((c, h, w)).astype(np.float32)
        col = ob.im2col(im, k, s, p)
        oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
        assert col.shape == (c * k * k, oh * ow)
        for ci in range(c):
            for i in range(k):
                for j in range(k):
                    for y in range(oh):
                        for x in range(ow):
                            yy, xx = y * s + i - p, x * s + j - p
                            want = im[ci, yy, xx] if 0 <= yy < h and 0 <= xx < w else 0.0
                            assert col[(ci * k + i) * k + j, y * ow + x] == want


@pytest.mark.parametrize("geom", [(2, 3, 12, 12, 5, 3, 1, 1), (2, 4, 15, 13, 6, 5, 2, 2), (1, 3, 23, 23, 4, 11, 4, 0),
                                  (3, 8, 7, 7, 16, 1, 1, 0), (2, 3, 14, 14, 4, 7, 2, 3)])
def test_conv_equals_cross_correlation(geom):
    B, Cc, H, W, Fo, k, s, p = geom
    rng = np.random.default_rng(sum(geom))
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    w = (rng.standard_normal((Fo, Cc, k, k)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Fo).astype(np.float32)
    got = ob.conv_forward(x, w, b, None, s, p, "linear")
    want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(),
                    stride=s, padding=p).numpy()
    assert got.shape == want.shape
    assert rel(got, want) < 1e-5


def test_conv_bn_is_affine_with_eps_outside_root():
    # y = bias + scale * (conv - mean) / (sqrt(var) + 1e-5); a small variance makes eps placement visible
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 3, 8, 8)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    scale = rng.uniform(0.8, 1.2, 4).astype(np.float32)
    mean = (rng.standard_normal(4) * 0.1).astype(np.float32)
    var = np.array([1e-6, 4e-6, 1.0, 0.5], np.float32)
    got = ob.conv_forward(x, w, bias, (scale, mean, var), 1, 1, "linear").astype(np.float64)
    raw = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), None, padding=1).numpy()
    sh = (1, 4, 1, 1)
    outside = (raw - mean.reshape(sh)) / (np.sqrt(var.astype(np.float64)).reshape(sh) + 1e-5) * scale.reshape(sh) \
        + bias.reshape(sh)
    inside = (raw - mean.reshape(sh)) / np.sqrt(var.astype(np.float64) + 1e-5).reshape(sh) * scale.reshape(sh) \
        + bias.reshape(sh)
    assert rel(got, outside) < 1e-5
    assert rel(got, inside) > 1e-2      # the other placement is far away for var ~ 1e-6


def test_connected_is_x_times_w_transposed():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 3, 4, 5)).astype(np.float32)     # NCHW flatten
    w = rng.standard_normal((11, 60)).astype(np.float32)
    b = rng.standard_normal(11).astype(np.float32)
    got = ob.connected_forward(x, w, b, None, "linear")
    want = x.reshape(7, 60).astype(np.float64) @ w.astype(np.float64).T + b
    assert rel(got, want) < 1e-5


def test_maxpool_equals_torch_when_window_equals_stride():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 3, 12, 12)).astype(np.float32)
    y, idx = ob.maxpool_forward(x, 2, 2, 0)
    ty, tidx = F.max_pool2d(torch.from_numpy(x), 2, 2, return_indices=True)
    np.testing.assert_array_equal(y, ty.numpy())
    # torch indexes within one (b, c) plane; the reference stores the offset into the whole tensor
    plane = np.arange(6).reshape(2, 3, 1, 1) * 144
    np.testing.assert_array_equal(idx, (tidx.numpy() + plane).astype(np.uint32))
    # and the index really addresses the maximum
    np.testing.assert_array_equal(x.ravel()[idx.ravel()], y.ravel())


def test_maxpool_k3s2_and_size_rule():
    # AlexNet chain 55 -> 27 -> 13 -> 6 with padding 0 and ResNet 112 -> 56 (out = (in + 2p) / stride)
    assert [ob.pool_out_dim(n, 2, 0) for n in (55, 27, 13, 112)] == [27, 13, 6, 56]
    assert ob.oracle().orc_pool_default_padding(3) == 1 and ob.oracle().orc_pool_default_padding(2) == 0
    rng = np.random.default_rng(7)
    x = rng.standard_normal((1, 2, 11, 11)).astype(np.float32)
    y, idx = ob.maxpool_forward(x, 3, 2, 0)      # 11 -> 5, every window inside the image
    ty = F.max_pool2d(torch.from_numpy(x), 3, 2)
    np.testing.assert_array_equal(y, ty.numpy())
    # first maximum wins on ties (row-major scan of the window)
    x2 = np.zeros((1, 1, 4, 4), np.float32)
    _, idx2 = ob.maxpool_forward(x2, 2, 2, 0)
    np.testing.assert_array_equal(idx2.ravel(), [0, 2, 8, 10])


def test_avgpool_counts_padding():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 2, 8, 8)).astype(np.float32)
    got = ob.avgpool_forward(x, 3, 2, 1)        # (8 + 2) / 2 = 5 outputs; the last window hangs off the edge
    padded = np.zeros((2, 2, 12, 12), np.float64)
    padded[:, :, 1:9, 1:9] = x
    want = np.zeros((2, 2, 5, 5))
    for h in range(5):
        for w in range(5):
            want[:, :, h, w] = padded[:, :, 2 * h:2 * h + 3, 2 * w:2 * w + 3].sum(axis=(2, 3)) / 9.0
    assert rel(got, want) < 1e-6
    glob = ob.avgpool_forward(x[:, :, :7, :7], 7, 7, 0)
    assert rel(glob.reshape(2, 2), x[:, :, :7, :7].astype(np.float64).mean(axis=(2, 3))) < 1e-6


def test_shortcut_invariants():
    rng = np.random.default_rng(9)
    a = rng.standard_normal((2, 4, 6, 6)).astype(np.float32)
    b = rng.standard_normal((2, 4, 6, 6)).astype(np.float32)
    np.testing.assert_array_equal(ob.shortcut_forward(b, a), a + b)           # same shape: plain add
    wide = rng.standard_normal((2, 16, 6, 6)).astype(np.float32)
    out = ob.shortcut_forward(wide, a)                                         # channel growth
    np.testing.assert_array_equal(out[:, :4], wide[:, :4] + a)
    np.testing.assert_array_equal(out[:, 4:], wide[:, 4:])
    small = rng.standard_normal((2, 8, 3, 3)).astype(np.float32)
    out = ob.shortcut_forward(small, a)                                        # 6 -> 3: conn[::2, ::2]
    np.testing.assert_array_equal(out[:, :4], small[:, :4] + a[:, :, ::2, ::2])
    odd = rng.standard_normal((1, 2, 19, 19)).astype(np.float32)
    tgt = rng.standard_normal((1, 2, 10, 10)).astype(np.float32)
    out = ob.shortcut_forward(tgt, odd)                                        # 19 / 10 = 1: top-left crop
    np.testing.assert_array_equal(out, tgt + odd[:, :, :10, :10])
    relu = ob.shortcut_forward(b, a, "relu")
    np.testing.assert_array_equal(relu, np.maximum(a + b, 0))


def test_softmax_properties():
    rng = np.random.default_rng(10)
    x = (rng.standard_normal((5, 1000)) * 4).astype(np.float32)
    y = ob.softmax_forward(x)
    assert np.abs(y.sum(axis=1) - 1).max() < 1e-5
    assert rel(y, torch.softmax(torch.from_numpy(x).double(), 1).numpy()) < 1e-5
    shifted = ob.softmax_forward(x + np.float32(8.0))
    assert rel(shifted, y) < 1e-5
    assert (y.argmax(1) == x.argmax(1)).all()


def test_activation_closed_forms():
    x = np.linspace(-6, 6, 2001).astype(np.float32)
    d = x.astype(np.float64)
    assert rel(ob.activate("logistic", x), 1 / (1 + np.exp(-d))) < 1e-6
    assert rel(ob.activate("tanh", x), np.tanh(d)) < 1e-6
    assert rel(ob.activate("loggy", x), 2 / (1 + np.exp(-d)) - 1) < 1e-6
    np.testing.assert_array_equal(ob.activate("relu", x), np.maximum(x, 0))
    np.testing.assert_array_equal(ob.activate("leaky", x), np.where(x > 0, x, (0.1 * d).astype(np.float32)))
    np.testing.assert_array_equal(ob.activate("relie", x), np.where(x > 0, x, (0.01 * d).astype(np.float32)))
    np.testing.assert_array_equal(ob.activate("linear", x), x)
    # the three that differ from the textbook: squares, and 0/1 indicators
    np.testing.assert_array_equal(ob.activate("elu", x)[x > 0], (x * x)[x > 0])
    np.testing.assert_array_equal(ob.activate("hardtan", x), ((x > -1) & (x < 1)).astype(np.float32))
    np.testing.assert_array_equal(ob.activate("lhtan", x), ((x > 0) & (x < 1)).astype(np.float32))


def test_lstm_equals_torch_lstm():
    # standard cell, two bias vectors, no peepholes.  File order iW,fW,oW,cW,iU,fU,oU,cU; torch packs i,f,g,o.
    rng = np.random.default_rng(12)
    T, B, I, H = 5, 3, 7, 6
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    names = ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU")
    wt = {n: (rng.standard_normal((H, H if n[1] == "W" else I)) * 0.4).astype(np.float32) for n in names}
    bs = {n: (rng.standard_normal(H) * 0.3).astype(np.float32) for n in names}
    y, cell = ob.lstm_forward(x, [wt[n] for n in names], [bs[n] for n in names], want_cell=True)
    lstm = torch.nn.LSTM(I, H).double()
    with torch.no_grad():
        lstm.weight_ih_l0.copy_(torch.from_numpy(np.concatenate([wt["iU"], wt["fU"], wt["cU"], wt["oU"]])))
        lstm.weight_hh_l0.copy_(torch.from_numpy(np.concatenate([wt["iW"], wt["fW"], wt["cW"], wt["oW"]])))
        lstm.bias_ih_l0.copy_(torch.from_numpy(np.concatenate([bs["iU"], bs["fU"], bs["cU"], bs["oU"]])))
        lstm.bias_hh_l0.copy_(torch.from_numpy(np.concatenate([bs["iW"], bs["fW"], bs["cW"], bs["oW"]])))
        ty, (hn, cn) = lstm(torch.from_numpy(x).double())
    assert rel(y, ty.numpy()) < 1e-5
    assert rel(cell[-1], cn[0].numpy()) < 1e-5


def test_openblas_backend_matches_custom_gemm():
    if not ob.use_openblas(threads=2):
        pytest.skip("no OpenBLAS found")
    try:
        rng = np.random.default_rng(13)
        x = rng.standard_normal((2, 5, 14, 14)).astype(np.float32)
        w = (rng.standard_normal((7, 5, 3, 3)) * 0.2).astype(np.float32)
        b = rng.standard_normal(7).astype(np.float32)
        fast = ob.conv_forward(x, w, b, None, 1, 1, "relu")
        ob.use_custom_gemm()
        slow = ob.conv_forward(x, w, b, None, 1, 1, "relu")
        assert rel(fast, slow) < 1e-5
    finally:
        ob.use_custom_gemm()
        ob.set_threads(1)


def test_image_input_contract_closed_form_and_resize_bounds():
    """Byte -> plane conversion is a closed form; the resize restatement (parity unpinned: OpenCV is absent) must
    at least be the identity at equal size, keep constants, and stay within one grey level of exact bilinear
    interpolation with pixel-centre alignment (torch, align_corners=False, no antialias)."""
    rng = np.random.default_rng(3)
    img = rng.integers(0, 256, (13, 17, 3), dtype=np.uint8)
    got = ob.image_to_input(img, 13, 17)
    want = (img.astype(np.float64) / 255.0).astype(np.float32).transpose(2, 0, 1)[[2, 1, 0]]
    np.testing.assert_array_equal(got.view(np.uint32), np.ascontiguousarray(want).view(np.uint32))
    np.testing.assert_array_equal(ob.resize_linear_u8(img, 13, 17), img)
    const = np.full((9, 11, 3), 137, np.uint8)
    np.testing.assert_array_equal(ob.resize_linear_u8(const, 20, 7), np.full((20, 7, 3), 137, np.uint8))
    for (h, w, dh, dw) in [(13, 17, 26, 34), (40, 30, 16, 12), (31, 29, 47, 18), (8, 8, 227, 227), (64, 48, 5, 5)]:
        src = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
        got = ob.resize_linear_u8(src, dh, dw).astype(np.float64)
        t = torch.from_numpy(src.astype(np.float64)).permute(2, 0, 1)[None]
        exact = torch.nn.functional.interpolate(t, size=(dh, dw), mode="bilinear", align_corners=False, antialias=False)
        exact = exact[0].permute(1, 2, 0).numpy()
        assert np.abs(got - exact).max() <= 1.0 + 1e-9, (h, w, dh, dw, np.abs(got - exact).max())
        assert np.abs(got - exact).mean() < 0.35
    gray = rng.integers(0, 256, (10, 12, 1), dtype=np.uint8)
    np.testing.assert_array_equal(ob.image_to_input(gray, 10, 12)[0], (gray[..., 0] / 255.0).astype(np.float32))


def _exact_taps(dst_n, src_n, clamp_weight):
    """Source index and weights of the pixel-centre mapping x = (d + 1/2) * src/dst - 1/2, from exact fractions."""
    from fractions import Fraction
    ofs, w, tie = [], [], []
    for d in range(dst_n):
        x = Fraction(2 * d + 1, 2) * Fraction(src_n, dst_n) - Fraction(1, 2)
        s = x.numerator // x.denominator            # floor, also for negatives
        f = x - s
        if clamp_weight and s < 0:
            s, f = 0, Fraction(0)
        if clamp_weight and s >= src_n - 1:
            s, f = src_n - 1, Fraction(0)
        ofs.append(s)
        w.append(f * 2048)
        tie.append((f * 4096).denominator == 1 and (f * 2048).denominator != 1)
    return ofs, w, tie


@pytest.mark.parametrize("dst_n,src_n", [(8, 8), (16, 8), (8, 16), (24, 8), (8, 24), (32, 8), (227, 256), (224, 500), (224, 375), (47, 31),
                                         (5, 64), (227, 8), (12, 30), (3, 2), (2, 3), (1, 7), (7, 1)])
@pytest.mark.parametrize("clamp_weight", [0, 1])
def test_resize_tap_table_against_rational_closed_form(dst_n, src_n, clamp_weight):
    """The table of the resize restatement holds, per destination pixel, floor(x) and the weights (1 - f, f) * 2048 rounded
    to the nearest integer, x being the exact rational pixel-centre coordinate; the two weights always add up to 2048.
    A shifted mapping (corner alignment, a dropped half pixel), a swapped weight pair or a different scale fails here."""
    ofs, w = ob.linear_taps(dst_n, src_n, clamp_weight)
    want_ofs, want_w1, tie = _exact_taps(dst_n, src_n, clamp_weight)
    np.testing.assert_array_equal(ofs, np.array(want_ofs, np.int32))
    np.testing.assert_array_equal(w.astype(np.int64).sum(axis=1), np.full(dst_n, 2048))
    for d in range(dst_n):
        # the coordinate is held in float (as OpenCV holds it): its fraction is good to src_n * 2^-24
        assert abs(float(w[d, 1]) - float(want_w1[d])) <= 0.5 + 2048 * max(src_n, 1) * 2.0 ** -23, (d, w[d], want_w1[d])
        if want_w1[d].denominator == 1:
            assert int(w[d, 1]) == int(want_w1[d])
        if tie[d]:                                  # an exact half rounds to the even neighbour
            assert int(w[d, 1]) % 2 == 0


def test_resize_exact_halving_is_the_rounded_box_mean():
    """At exactly half size every weight is 1024/2048 and the fixed-point passes lose nothing:
    dst = (a + b + c + d + 2) >> 2 over each 2x2 block, the result OpenCV's own 2x2 area path gives for this ratio."""
    rng = np.random.default_rng(11)
    for (h, w, c) in [(8, 10, 3), (64, 48, 1), (454, 454, 3), (2, 2, 4)]:
        src = rng.integers(0, 256, (h, w, c), dtype=np.uint8)
        s = src.astype(np.int64)
        want = (s[0::2, 0::2] + s[0::2, 1::2] + s[1::2, 0::2] + s[1::2, 1::2] + 2) >> 2
        np.testing.assert_array_equal(ob.resize_linear_u8(src, h // 2, w // 2), want.astype(np.uint8))
        ofs, wt = ob.linear_taps(w // 2, w, 1)
        np.testing.assert_array_equal(ofs, 2 * np.arange(w // 2))
        assert (wt == 1024).all()
    extremes = np.zeros((4, 4, 1), np.uint8); extremes[:2] = 255
    np.testing.assert_array_equal(ob.resize_linear_u8(extremes, 2, 2)[..., 0], [[255, 255], [0, 0]])


def test_resize_exact_doubling_is_the_quarter_stencil():
    """At exactly double size the taps are 1/4 : 3/4 (512 / 1536 of 2048), with the border pixel repeated.  On ramps
    whose steps are multiples of 16 no intermediate is rounded, so the output is the stencil's exact value; an impulse
    returns the separable response [1, 3, 3, 1] x [1, 3, 3, 1] / 16 with the scheme's truncations."""
    ofs, wt = ob.linear_taps(16, 8, 1)
    np.testing.assert_array_equal(ofs, [0, 0, 0, 1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6, 7])
    np.testing.assert_array_equal(wt[:, 1], [0] + [512, 1536] * 7 + [0])
    ofs, wt = ob.linear_taps(16, 8, 0)                       # rows: weights stay, the row index is clipped later
    np.testing.assert_array_equal(ofs, [-1] + [k // 2 for k in range(15)])
    np.testing.assert_array_equal(wt[:, 1], [1536, 512] * 8)

    def stencil(v):                                          # exact 1-D doubling of an integer sequence, times 4
        p = np.concatenate([v[:1], v, v[-1:]]).astype(np.int64)
        out = np.empty(2 * len(v), np.int64)
        out[0::2] = p[:-2] + 3 * p[1:-1]
        out[1::2] = 3 * p[1:-1] + p[2:]
        return out
    xs = 16 * np.arange(12)
    ys = 16 * np.arange(9)
    ramp = (xs[None, :] + ys[:, None])
    ramp = np.where(ramp > 240, 480 - ramp, ramp).astype(np.uint8)      # a ridge, still piecewise linear in steps of 16
    hor = np.stack([stencil(r) for r in ramp.astype(np.int64)])         # times 4
    both = np.stack([stencil(col) for col in hor.T]).T                  # times 16
    assert (both % 16 == 0).all()
    np.testing.assert_array_equal(ob.resize_linear_u8(ramp[..., None], 18, 24)[..., 0], (both // 16).astype(np.uint8))

    imp = np.zeros((6, 7, 1), np.uint8); imp[2, 3] = 255
    got = ob.resize_linear_u8(imp, 12, 14)[..., 0].astype(np.int64)
    k = np.array([1, 3, 3, 1])
    exact = 255 * np.outer(k, k) / 16.0
    blk = got[3:7, 5:9]
    assert np.abs(blk - exact).max() < 1.0 and got.sum() == blk.sum()
    np.testing.assert_array_equal(blk, blk.T)
    np.testing.assert_array_equal(blk, blk[::-1, ::-1])
    # the scheme itself on this block: horizontal sums 255 * {512, 1536}, >> 4, times the row weight, >> 16, + 2 >> 2
    h4 = 255 * np.array([512, 1536, 1536, 512])
    fixed = ((((np.array([512, 1536, 1536, 512])[:, None] * (h4[None, :] >> 4)) >> 16) + 2) >> 2)
    np.testing.assert_array_equal(blk, fixed)
