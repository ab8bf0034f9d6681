"""The benchmarked configurations (AlexNet, VGG-16, ResNet-50, the two-layer LSTM) at their real layer shapes.  Against the oracle (OpenBLAS backend, so it
finishes in seconds) at a batch the CPU can afford, and at the full batch through properties that do
not depend on size: per-image independence, argmax addressing the maximum, linearity."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import bench  # noqa: E402  (synthetic weight generator shared with the benchmark)
from nebula_amd import zoo  # noqa: E402
from oracle import binding as ob  # noqa: E402

TOL = 1e-4


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


def build(cfg, wdist="he", seed=5):
    from nebula_amd.net import Network
    net = Network(cfg)
    blob = bench.make_weights(net.weight_layout(), np.random.default_rng(seed), wdist)
    net.load_weight_blob(blob)
    return net, blob


def oracle_forward(cfg, blob, x):
    assert ob.use_openblas(threads=16)
    try:
        onet = ob.OracleNet(cfg)
        onet.load_weights(blob)
        return onet.forward(x)
    finally:
        ob.use_custom_gemm()
        ob.set_threads(1)


def test_config1_conv1_relu_maxpool_full_size():
    print("CASE config 1 full size", flush=True)
    cfg = zoo.conv1_pool_cfg(32, pool_index=True)
    rng = np.random.default_rng(1)
    x = rng.random((32, 3, 227, 227), dtype=np.float32)
    net, blob = build(cfg)
    want = oracle_forward(cfg, blob, x)
    net.set_input(x)
    net.forward()
    conv = net.output(0).reshape(32, 96, 55, 55)
    assert rel(conv, want[0]) <= TOL
    # pooling is exact on identical input: pool the GPU's own conv output on the CPU
    py, pidx = ob.maxpool_forward(conv, 3, 2, 0)
    np.testing.assert_array_equal(net.output(1).view(np.uint32), py.ravel().view(np.uint32))
    np.testing.assert_array_equal(net.pool_index(1), pidx.ravel())
    # relu mask: exact wherever the pre-activation is clear of zero
    assert (conv >= 0).all()
    net.close()


@pytest.mark.parametrize("name,batch", [("resnet50", 2), ("alexnet", 4), ("vgg16", 1)])
def test_image_networks_against_oracle(name, batch):
    print("CASE", name, "vs oracle at batch", batch, flush=True)
    cfg = zoo.WORKLOADS[name](batch)
    rng = np.random.default_rng(2)
    net, blob = build(cfg)
    c, h, w = net.input_shape
    x = (rng.random((batch, c, h, w)) if name == "alexnet" else rng.standard_normal((batch, c, h, w))).astype(np.float32)
    want = oracle_forward(cfg, blob, x)
    net.set_input(x)
    net.forward()
    kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
    logits_at = max(i for i, k in enumerate(kinds) if k == "connected_layer")
    worst = 0.0
    for i, k in enumerate(kinds):
        if k in ("cost_layer", "dropout_layer"):
            continue
        r = rel(net.output(i), want[i].ravel())
        worst = max(worst, r)
        assert r <= TOL, (name, i, k, r)
    got, ref = net.output(logits_at).reshape(batch, -1), want[logits_at].reshape(batch, -1)
    np.testing.assert_array_equal(got.argmax(1), ref.argmax(1))
    top2 = np.sort(ref, axis=1)[:, -2:]
    print("   worst layer rel err %.2e, min top-1/top-2 margin %.3e" % (worst, float((top2[:, 1] - top2[:, 0]).min())), flush=True)
    net.close()


def test_lstm_full_width_against_oracle():
    print("CASE lstm 1024/1024 vs oracle", flush=True)
    T, B = 4, 64
    cfg = zoo.lstm_cfg(batch=B, time_steps=T, classes=1000, last_step_only=True)
    rng = np.random.default_rng(3)
    net, blob = build(cfg, "lstm")
    x = rng.standard_normal((T, B, 1024)).astype(np.float32)
    want = oracle_forward(cfg, blob, x)
    net.set_input(x)
    net.forward()
    for i in (0, 1):
        assert rel(net.output(i), want[i].ravel()) <= TOL
    probs = net.output(3).reshape(T * B, -1)[:B]
    assert rel(probs, want[3]) <= TOL
    np.testing.assert_array_equal(probs.argmax(1), want[3].argmax(1))
    net.close()


def test_resnet50_batch64_images_are_independent():
    """Headline configuration: every image of the batch-64 run must equal the same image run at batch 2
    (inference has no cross-image term), up to the reassociation different tile shapes may cause."""
    print("CASE resnet50 b64 independence", flush=True)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((64, 3, 224, 224)).astype(np.float32)
    net64, blob = build(zoo.resnet50_cfg(64))
    net64.set_input(x)
    net64.forward()
    last = net64.num_layers - 3          # connected layer (then softmax, cost)
    assert net64.layer_info(last)["kind"] == "connected_layer"
    logits64 = net64.output(last).reshape(64, 1000)
    probs64 = net64.output(last + 1).reshape(64, 1000)
    net64.close()
    net2, _ = build(zoo.resnet50_cfg(2))
    for lo in (0, 62):
        net2.set_input(x[lo:lo + 2])
        net2.forward()
        logits2 = net2.output(last).reshape(2, 1000)
        assert rel(logits64[lo:lo + 2], logits2) <= TOL
        np.testing.assert_array_equal(logits64[lo:lo + 2].argmax(1), logits2.argmax(1))
    net2.close()
    assert np.isfinite(logits64).all()
    assert np.abs(probs64.sum(1) - 1).max() < 1e-4


def test_full_size_maxpool_and_conv_properties():
    from nebula_amd import hip
    print("CASE full-size properties", flush=True)
    ctx = hip.Ctx(0)
    rng = np.random.default_rng(6)
    # ResNet's maxpool at batch 64: the stored index addresses the maximum, which is one of the taps
    x = rng.standard_normal((64, 64, 112, 112)).astype(np.float32)
    y, idx = ctx.pool(ctx.array(x), 3, 2, 0, "max")
    y, idx = y.numpy(), idx.numpy()
    np.testing.assert_array_equal(x.ravel()[idx.ravel()], y.ravel())
    win = np.lib.stride_tricks.sliding_window_view(x[:2], (3, 3), axis=(2, 3))[:, :, ::2, ::2]   # [2,64,55,55,3,3]
    np.testing.assert_array_equal(win.max(axis=(4, 5)), y[:2, :, :55, :55])
    # a ResNet stage-3 3x3 convolution at batch 64: linear in its input (no bias, linear activation)
    w = (rng.standard_normal((128, 128, 3, 3)) * 0.03).astype(np.float32)
    plan = ctx.conv_pack(w, np.zeros(128, np.float32), None, H=28, W=28, stride=1, pad=1, act="linear")
    a = rng.standard_normal((64, 128, 28, 28)).astype(np.float32)
    b = rng.standard_normal((64, 128, 28, 28)).astype(np.float32)
    ya, yb, yab = plan(ctx.array(a)).numpy(), plan(ctx.array(b)).numpy(), plan(ctx.array(a + 2 * b)).numpy()
    assert rel(yab, ya + 2 * yb) <= TOL
    # and a spot check of 3 images against the oracle
    want = ob.conv_forward(a[[0, 31, 63]], w, np.zeros(128, np.float32), None, 1, 1, "linear")
    assert rel(ya[[0, 31, 63]], want) <= TOL
    ctx.close()
