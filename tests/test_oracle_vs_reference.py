"""The CPU oracle against the compiled, unmodified reference (oracle/_ref/libnebula_ref.so) on
seeded random inputs.  That library can only be built where the reference tree exists, so these
tests skip elsewhere (the committed golden vectors cover the same ground there)."""
import os

import numpy as np
import pytest

from oracle import binding as ob

# decided from the tree alone: nothing is compiled or loaded while pytest collects, and nothing at all where the
# reference is absent
pytestmark = pytest.mark.skipif(not os.path.isdir(ob.REFERENCE_ROOT), reason="reference tree not present")


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


@pytest.mark.parametrize("shape", [(3, 9, 9, 3, 1, 1), (2, 11, 7, 5, 2, 2), (1, 35, 35, 11, 4, 0), (4, 6, 8, 1, 1, 0),
                                   (2, 8, 8, 3, 2, 1), (1, 7, 7, 7, 2, 3)])
def test_im2col(shape):
    c, h, w, k, s, p = shape
    rng = np.random.default_rng(sum(shape))
    im = rng.standard_normal((c, h, w)).astype(np.float32)
    got = ob.im2col(im, k, s, p)
    want = np.full_like(got, 7.0)
    ob.ref().ref_im2col(ob._fp(im), c, h, w, k, s, p, ob._fp(want), 2)
    np.testing.assert_array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm(ta, tb):
    rng = np.random.default_rng(5 + 2 * ta + tb)
    M, N, K = 13, 17, 29
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    ob.use_custom_gemm()
    got = ob.gemm(ta, tb, A, B, C0, alpha=0.75, beta=0.5)
    want = C0.copy()
    ob.ref().ref_gemm(ta, tb, M, N, K, 0.75, ob._fp(A), A.shape[1], ob._fp(B), B.shape[1], 0.5, ob._fp(want), N, 3)
    np.testing.assert_array_equal(bits(got), bits(want))


def test_batchnorm_bias_bit_exact():
    rng = np.random.default_rng(11)
    B, Cc, S = 5, 37, 41
    y = rng.standard_normal((B, Cc, S)).astype(np.float32)
    mean = (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    var = rng.uniform(0.01, 3.0, Cc).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, Cc).astype(np.float32)
    bias = rng.standard_normal(Cc).astype(np.float32)
    a, b = y.copy(), y.copy()
    o, r = ob.oracle(), ob.ref()
    o.orc_batchnorm_normalize(ob._fp(a), ob._fp(mean), ob._fp(var), Cc, S, B)
    r.ref_batchnorm_normalize(2, ob._fp(b), ob._fp(mean), ob._fp(var), Cc, S, B)
    np.testing.assert_array_equal(bits(a), bits(b))
    o.orc_batchnorm_scale_down(ob._fp(a), ob._fp(scale), Cc, S, B)
    r.ref_batchnorm_scale_down(2, ob._fp(b), ob._fp(scale), Cc, S, B)
    np.testing.assert_array_equal(bits(a), bits(b))
    o.orc_forward_bias(ob._fp(a), ob._fp(bias), Cc, S, B)
    r.ref_forward_bias(2, ob._fp(b), ob._fp(bias), Cc, S, B)
    np.testing.assert_array_equal(bits(a), bits(b))


@pytest.mark.parametrize("name", ob.ACT_NAMES[1:])
def test_activation(name):
    rng = np.random.default_rng(ob.ACT[name])
    x = np.concatenate([rng.standard_normal(50000) * 4, rng.uniform(-10, 10, 50000),
                        np.arange(-9, 9.5, 0.5)]).astype(np.float32)
    got = ob.activate(name, x)
    want = x.copy()
    assert ob.ref().ref_activation(ob.ACT[name], ob._fp(want), want.size) == 0
    np.testing.assert_array_equal(bits(got), bits(want))


@pytest.mark.parametrize("dims", [((2, 4, 9, 9), (2, 16, 9, 9)), ((2, 8, 10, 10), (2, 16, 5, 5)),
                                  ((1, 6, 19, 19), (1, 6, 10, 10)), ((2, 8, 4, 4), (2, 4, 8, 8)),
                                  ((3, 5, 7, 7), (3, 5, 7, 7))])
def test_shortcut_primitive(dims):
    conn_shape, out_shape = dims
    rng = np.random.default_rng(3)
    conn = rng.standard_normal(conn_shape).astype(np.float32)
    prev = rng.standard_normal(out_shape).astype(np.float32)
    got = ob.shortcut_forward(prev, conn, "linear")
    want = prev.copy()
    ob.ref().ref_shortcut(2, conn_shape[3], conn_shape[2], conn_shape[1], ob._fp(conn),
                          out_shape[3], out_shape[2], out_shape[1], ob._fp(want), out_shape[0])
    np.testing.assert_array_equal(bits(got), bits(want))


POOL_CFG = """
[net]
batch=%d
height=%d
width=%d
channels=%d
num_threads=2
[%s]
%s
"""


@pytest.mark.parametrize("kind", ["maxpool", "avgpool"])
@pytest.mark.parametrize("geom", [(2, 3, 12, 12, "size=3\nstride=2"), (2, 2, 13, 11, "size=3\nstride=2\npadding=0"),
                                  (1, 4, 8, 8, "stride=2"), (2, 2, 7, 7, "size=7\nstride=7\npadding=0"),
                                  (1, 2, 9, 9, "size=2\nstride=1\npadding=1"), (1, 1, 6, 6, "size=5\nstride=3")])
def test_pooling_layer(kind, geom):
    B, Cc, H, W, body = geom
    cfg = POOL_CFG % (B, H, W, Cc, kind, body)
    rng = np.random.default_rng(B * 100 + H)
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    x[0, 0, :2, :2] = 0.25           # ties: the first maximum must win
    rn = ob.RefNet(cfg)
    want = rn.forward(x)[0]
    net = ob.OracleNet(cfg)
    got = net.forward(x)[0]
    d = rn.layer_dims(0)
    assert got.shape == (B, d["output_channel"], d["output_height"], d["output_width"])
    np.testing.assert_array_equal(bits(got), bits(want))
    if kind == "maxpool":
        np.testing.assert_array_equal(net.specs[0].last_index.ravel(), rn.pool_index(0))


def test_maxpool_all_below_sentinel():
    # nothing beats the -1e8 sentinel -> value -1e8, index -1 (0xffffffff)
    cfg = POOL_CFG % (1, 4, 4, 1, "maxpool", "size=2\nstride=2\npadding=0")
    x = np.full((1, 1, 4, 4), -3e8, np.float32)
    rn = ob.RefNet(cfg)
    want = rn.forward(x)[0]
    y, idx = ob.maxpool_forward(x, 2, 2, 0)
    np.testing.assert_array_equal(bits(y), bits(want))
    np.testing.assert_array_equal(idx.ravel(), rn.pool_index(0))
    assert (idx == 0xFFFFFFFF).all()


def test_softmax_layer():
    cfg = "[net]\nbatch=6\nheight=1\nwidth=1\nchannels=333\n[softmax]\n"
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((6, 333, 1, 1)) * 5).astype(np.float32)
    want = ob.RefNet(cfg).forward(x)[0]
    got = ob.softmax_forward(x.reshape(6, 333))
    np.testing.assert_array_equal(bits(got), bits(want))


def test_cfg_parser_quirks():
    # upper-case keys/values are lowered, spaces stripped, unknown keys ignored, first duplicate wins
    cfg = "[net]\nBATCH = 2\nheight=5\nwidth=5\nchannels=2\nbogus=1\n[Convolutional]\n".lower() + \
          "FILTERS=3\nsize = 3\nSTRIDE=1\npadding=1\nACTIVATION=ReLU\nfilters=9\n"
    rn = ob.RefNet(cfg)
    net, specs = ob.plan_network(cfg)
    d = rn.layer_dims(0)
    assert (d["output_channel"], d["output_height"], d["output_width"]) == specs[0].out == (3, 5, 5)
    assert d["activation_type"] == ob.ACT["relu"]
