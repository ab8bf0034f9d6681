"""The CPU oracle against the committed golden vectors (tests/golden/*.npz), which were written
by tests/golden/make_golden.py from the compiled, unmodified reference (CUSTOM_BLAS build).
The oracle's default GEMM restates that same loop nest, so every layer output must match
bit for bit; so must the maxpool argmax tables."""
import glob
import os

import numpy as np
import pytest

from oracle import binding as ob

NETS = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))
              if not p.endswith("activations.npz"))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


def test_fixtures_present():
    assert {"alexnet_conv1_small", "convnet_mixed", "resnet_shortcuts", "lstm_plain", "lstm_bn_tanh",
            "rnn_plain", "rnn_bn_leaky", "dbn_small"} <= set(NETS)


@pytest.mark.parametrize("name", NETS)
@pytest.mark.parametrize("threads", [1, 3])
def test_network_layers_bit_exact(golden_dir, name, threads):
    g = np.load(os.path.join(golden_dir, name + ".npz"))
    cfg = str(g["cfg"])
    ob.use_custom_gemm()
    ob.set_threads(threads)
    net = ob.OracleNet(cfg)
    net.load_weights(g["weights"])
    T = net.net["time_steps"]
    if net.net["recurrent"]:
        x = g["input"].reshape(T, net.net["batch"], net.net["input_size"])
        assert int(g["batch_size"]) == T * net.net["batch"]      # recurrent.cc:139
    else:
        x = g["input"].reshape(net.net["batch"], net.net["channels"], net.net["height"], net.net["width"])
    outs = net.forward(x)
    for i, (sp, out) in enumerate(zip(net.specs, outs)):
        if sp.kind == "cost":
            continue
        want = g["out_%02d" % i]
        dims = g["dims_%02d" % i]
        assert out.size == want.size, (name, i, sp.kind, out.shape, want.shape)
        if sp.kind in ("convolutional", "maxpool", "avgpool", "shortcut"):
            assert tuple(out.shape[1:]) == (dims[0], dims[1], dims[2]), (name, i, sp.kind)
        np.testing.assert_array_equal(bits(out), bits(want), err_msg="%s layer %d (%s)" % (name, i, sp.kind))
        if sp.kind == "maxpool":
            np.testing.assert_array_equal(sp.last_index.ravel(), g["idx_%02d" % i])
    ob.set_threads(1)


def test_activations_bit_exact(golden_dir):
    g = np.load(os.path.join(golden_dir, "activations.npz"))
    x = g["input"]
    for name in ob.ACT_NAMES[1:]:
        got, want = ob.activate(name, x), g[name]
        same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), name


def test_activation_ids_rejected():
    x = np.zeros(4, np.float32)
    with pytest.raises(ValueError):
        ob.activate(0, x)       # UNDEFINED_ACTIVATION: layer.cc:102-107 exits
    with pytest.raises(ValueError):
        ob.activate(14, x)
