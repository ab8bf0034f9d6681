"""Whole cfg-described networks through the C++ layer framework (libnebula_layers.so, which calls
the C ABI) against the committed golden vectors of the reference and against the CPU oracle."""
import glob
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402

TOL = 1e-4
NETS = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))
              if not p.endswith("activations.npz"))


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


@pytest.mark.parametrize("name", NETS)
def test_golden_network(golden_dir, name):
    from nebula_amd.net import Network
    print("CASE golden network", name, flush=True)
    g = np.load(os.path.join(golden_dir, name + ".npz"))
    with Network(str(g["cfg"])) as net:
        assert net.batch_size == int(g["batch_size"]) and net.time_step == int(g["time_step"])
        net.load_weight_blob(g["weights"])
        net.set_input(g["input"])
        net.forward()
        for i in range(net.num_layers):
            info = net.layer_info(i)
            dims = g["dims_%02d" % i]
            assert info["output_size"] == dims[3], (name, i)
            assert info["layer_type"] == dims[4] and info["activation_type"] == dims[5], (name, i)
            if info["kind"] in ("convolutional_layer", "maxpool_layer", "avgpool_layer", "shortcut_layer"):
                assert (info["output_channel"], info["output_height"], info["output_width"]) == tuple(dims[:3])
            if info["kind"] == "cost_layer":
                continue
            got, want = net.output(i), g["out_%02d" % i]
            assert rel(got, want) <= TOL, (name, i, info["kind"], rel(got, want))
        last = [i for i in range(net.num_layers) if net.layer_info(i)["kind"] != "cost_layer"][-1]
        rows = net.batch_size
        got, want = net.output(last).reshape(rows, -1), g["out_%02d" % last].reshape(rows, -1)
        np.testing.assert_array_equal(got.argmax(1), want.argmax(1))


def test_maxpool_index_through_layer(golden_dir):
    # identical input to the pooling layer -> identical argmax table: feed the pool layer directly
    from nebula_amd.net import Network
    cfg = "[net]\nbatch=2\nheight=13\nwidth=11\nchannels=3\npool_index=1\n[maxpool]\nsize=3\nstride=2\n"
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 13, 11)).astype(np.float32)
    with Network(cfg) as net:
        net.set_input(x)
        net.forward()
        wy, widx = ob.maxpool_forward(x, 3, 2, 1)
        np.testing.assert_array_equal(net.output(0).view(np.uint32), wy.ravel().view(np.uint32))
        np.testing.assert_array_equal(net.pool_index(0), widx.ravel())
    # without the key the values are the same and the table is not kept
    from nebula_amd.net import NetworkError
    with Network(cfg.replace("pool_index=1\n", "")) as net:
        net.set_input(x)
        net.forward()
        np.testing.assert_array_equal(net.output(0).view(np.uint32), wy.ravel().view(np.uint32))
        with pytest.raises(NetworkError, match="pool_index=1"):
            net.pool_index(0)


def test_cfg_errors_are_reported():
    from nebula_amd.net import Network, NetworkError
    with pytest.raises(NetworkError, match="unknown layer type"):
        Network("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[bogus]\nx=1\n")
    with pytest.raises(NetworkError, match="undefined activation type"):
        Network("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[convolutional]\nfilters=2\nsize=3\nactivation=swish\n")
    with pytest.raises(NetworkError, match="invalid config"):
        Network("[net]\nbatch=1\nheight\n")
    with pytest.raises(NetworkError, match="failed to open"):
        Network("/nonexistent/network.cfg", is_text=False)
    with Network("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[connected]\noutput=3\nactivation=linear\n") as net:
        with pytest.raises(NetworkError, match="no weights"):
            net.forward()
        with pytest.raises(NetworkError, match="shorter"):
            net.load_weight_blob(np.zeros(5, np.float32))


def test_weights_round_trip(tmp_path, golden_dir):
    from nebula_amd.net import Network
    g = np.load(os.path.join(golden_dir, "convnet_mixed.npz"))
    with Network(str(g["cfg"])) as net:
        net.load_weight_blob(g["weights"])
        out = str(tmp_path / "out.wgh")
        assert __import__("nebula_amd.net", fromlist=["lib"]).lib().nbl_net_store_weights(net.h, out.encode()) == 0
        np.testing.assert_array_equal(np.fromfile(out, np.float32), g["weights"])


def _random_weights(specs, rng):
    parts = []
    for li, name, shape in ob.weight_layout(specs):
        base = name.split(".")[-1]
        if base == "weight":
            a = rng.standard_normal(shape) * np.sqrt(2.0 / int(np.prod(shape[1:])))
        elif base == "bias":
            a = rng.standard_normal(shape) * 0.1
        elif base == "scale":
            a = rng.uniform(0.8, 1.2, shape)
        elif base == "mean":
            a = rng.standard_normal(shape) * 0.1
        else:
            a = rng.uniform(0.5, 1.5, shape)
        parts.append(a.astype(np.float32).ravel())
    return np.concatenate(parts)


MINI_RESNET = """
[net]
batch=4
height=32
width=32
channels=3
[convolutional]
batch_normalize=1
filters=16
size=7
stride=2
padding=3
activation=relu
[maxpool]
size=3
stride=2
padding=0
""" + "".join("""
[convolutional]
batch_normalize=1
filters=%d
size=1
stride=1
padding=0
activation=relu
[convolutional]
batch_normalize=1
filters=%d
size=3
stride=%d
padding=1
activation=relu
[convolutional]
batch_normalize=1
filters=%d
size=1
stride=1
padding=0
activation=linear
[shortcut]
hops=4
activation=relu
""" % (c, c, s, 4 * c) for c, s in [(16, 1), (16, 1), (32, 2), (32, 1)]) + """
[avgpool]
size=4
stride=4
padding=0
[connected]
output=10
activation=linear
[softmax]
"""


def test_mini_resnet_against_oracle():
    from nebula_amd.net import Network
    print("CASE mini resnet", flush=True)
    rng = np.random.default_rng(42)
    onet = ob.OracleNet(MINI_RESNET)
    blob = _random_weights(onet.specs, rng)
    onet.load_weights(blob)
    x = rng.standard_normal((4, 3, 32, 32)).astype(np.float32)
    ob.use_custom_gemm()
    want = onet.forward(x)
    with Network(MINI_RESNET) as net:
        net.load_weight_blob(blob)
        net.set_input(x)
        net.forward()
        for i in range(net.num_layers):
            got = net.output(i)
            assert rel(got, want[i].ravel()) <= TOL, (i, net.layer_info(i)["kind"], rel(got, want[i].ravel()))
        logits = net.output(net.num_layers - 2).reshape(4, -1)
        np.testing.assert_array_equal(logits.argmax(1), want[-2].reshape(4, -1).argmax(1))


def test_lstm_last_step_only_against_oracle():
    from nebula_amd import zoo
    from nebula_amd.net import Network
    print("CASE lstm last_step_only", flush=True)
    T, B, I, H, Cn = 5, 6, 24, 64, 37
    rng = np.random.default_rng(8)
    for last in (False, True):
        cfg = zoo.lstm_cfg(batch=B, time_steps=T, input_size=I, hidden=H, layers=2, classes=Cn, last_step_only=last)
        onet = ob.OracleNet(cfg)
        blob = np.concatenate([rng.uniform(-1, 1, int(np.prod(sh))).astype(np.float32) / np.float32(np.sqrt(H))
                               for _, _, sh in ob.weight_layout(onet.specs)])
        onet.load_weights(blob)
        x = rng.standard_normal((T, B, I)).astype(np.float32)
        ob.use_custom_gemm()
        want = onet.forward(x)
        rows = B if last else T * B
        assert want[3].shape == (rows, Cn)
        with Network(cfg) as net:
            net.load_weight_blob(blob)
            net.set_input(x)
            net.forward()
            for i in (0, 1):
                assert rel(net.output(i), want[i].ravel()) <= TOL
            probs = net.output(3).reshape(T * B, Cn)[:rows]
            assert rel(probs, want[3]) <= TOL
            np.testing.assert_array_equal(probs.argmax(1), want[3].argmax(1))


@pytest.mark.parametrize("H", [128, 48])
def test_lstm_network_carries_state_between_batches_of_one_stream(H):
    """The reference's recurrent driver runs a token stream as consecutive batches of time_steps and its LSTM layers
    never clear their state in between (lstm_layer.cu:15-140).  [net] carry_state=1: two passes over the halves of a
    sequence give what the oracle gives for the whole sequence; reset_state starts a new stream; the default network
    starts every pass from zero."""
    from nebula_amd import zoo
    from nebula_amd.net import Network
    print("CASE lstm network carry_state", H, flush=True)
    T, B, I, Cn = 6, 5, 24, 19
    rng = np.random.default_rng(H)
    whole_cfg = zoo.lstm_cfg(batch=B, time_steps=T, input_size=I, hidden=H, layers=2, classes=Cn)
    half_cfg = zoo.lstm_cfg(batch=B, time_steps=T // 2, input_size=I, hidden=H, layers=2, classes=Cn)
    onet = ob.OracleNet(whole_cfg)
    blob = np.concatenate([rng.uniform(-1, 1, int(np.prod(sh))).astype(np.float32) / np.float32(np.sqrt(H))
                           for _, _, sh in ob.weight_layout(onet.specs)])
    onet.load_weights(blob)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    ob.use_custom_gemm()
    want = onet.forward(x)
    half_rows = T // 2 * B
    ohalf = ob.OracleNet(half_cfg)
    ohalf.load_weights(blob)
    want_fresh = ohalf.forward(x[T // 2:])               # the second half from zero state
    with Network(half_cfg.replace("[net]\n", "[net]\ncarry_state=1\nhip_graph=1\n", 1)) as net:
        net.load_weight_blob(blob)
        for rep in range(2):
            parts = []
            for part in (x[:T // 2], x[T // 2:]):
                net.set_input(part)
                net.forward()
                parts.append([net.output(i).copy() for i in range(4)])
            assert not net.graph_active                   # what a pass reads depends on the pass before it
            for i in (0, 1, 3):
                w = want[i].reshape(T * B, -1)
                assert rel(parts[0][i].reshape(half_rows, -1), w[:half_rows]) <= TOL, (rep, i)
                assert rel(parts[1][i].reshape(half_rows, -1), w[half_rows:]) <= TOL, (rep, i)
            assert rel(parts[1][1], want_fresh[1].ravel()) > 1e-3          # (the state does matter for these weights)
            net.reset_state()
        net.set_carry_state(False)
        net.set_input(x[T // 2:])
        net.forward()
        assert rel(net.output(1), want_fresh[1].ravel()) <= TOL
        net.forward()
        assert rel(net.output(1), want_fresh[1].ravel()) <= TOL
    with Network(half_cfg) as net:                          # the default: every pass from zero
        net.load_weight_blob(blob)
        for _ in range(2):
            net.set_input(x[T // 2:])
            net.forward()
            assert rel(net.output(3).reshape(half_rows, -1), want_fresh[3]) <= TOL


def test_fused_shortcut_is_bit_identical():
    """fuse_shortcut=1 moves the residual add into the convolution's epilogue: same operations, same order."""
    from nebula_amd.net import Network
    print("CASE fused shortcut", flush=True)
    rng = np.random.default_rng(17)
    # conv_split=0: one summation order whatever tile shape each network's search settles on
    plain_cfg = MINI_RESNET.replace("[net]\n", "[net]\nconv_split=0\n", 1)
    fused_cfg = plain_cfg.replace("[net]\n", "[net]\nfuse_shortcut=1\n", 1)
    onet = ob.OracleNet(MINI_RESNET)
    blob = _random_weights(onet.specs, rng)
    x = rng.standard_normal((4, 3, 32, 32)).astype(np.float32)
    outs = []
    for cfg in (plain_cfg, fused_cfg):
        with Network(cfg) as net:
            net.load_weight_blob(blob)
            net.set_input(x)
            net.forward()
            kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
            outs.append([net.output(i) for i in range(net.num_layers)])
    for i, k in enumerate(kinds):
        if k == "convolutional_layer" and i + 1 < len(kinds) and kinds[i + 1] == "shortcut_layer":
            # the fused convolution's output pointer aliases the shortcut's buffer
            np.testing.assert_array_equal(outs[1][i].view(np.uint32), outs[1][i + 1].view(np.uint32))
            continue
        np.testing.assert_array_equal(outs[0][i].view(np.uint32), outs[1][i].view(np.uint32), err_msg="layer %d %s" % (i, k))


def test_fused_shortcut_on_golden_resnet(golden_dir):
    from nebula_amd.net import Network
    g = np.load(os.path.join(golden_dir, "resnet_shortcuts.npz"))
    cfg = str(g["cfg"]).replace("[net]\n", "[net]\nfuse_shortcut=1\n", 1)
    with Network(cfg) as net:
        net.load_weight_blob(g["weights"])
        net.set_input(g["input"])
        net.forward()
        for i in range(net.num_layers):
            info = net.layer_info(i)
            nxt = net.layer_info(i + 1)["kind"] if i + 1 < net.num_layers else ""
            if info["kind"] == "convolutional_layer" and nxt == "shortcut_layer":
                continue
            assert rel(net.output(i), g["out_%02d" % i]) <= TOL, (i, info["kind"])


def test_network_input_from_byte_images():
    """set_input_images == set_input of the CPU-preprocessed batch (the image driver's load_data contract)."""
    from nebula_amd.net import Network
    print("CASE byte-image input", flush=True)
    rng = np.random.default_rng(23)
    onet = ob.OracleNet(MINI_RESNET)
    blob = _random_weights(onet.specs, rng)
    imgs = rng.integers(0, 256, (4, 45, 52, 3), dtype=np.uint8)
    x = np.stack([ob.image_to_input(im, 32, 32) for im in imgs])
    with Network(MINI_RESNET) as net:
        net.load_weight_blob(blob)
        net.set_input(x)
        net.forward()
        a = [net.output(i) for i in range(net.num_layers)]
        net.set_input(np.zeros_like(x))
        net.set_input_images(imgs)
        net.forward()
        b = [net.output(i) for i in range(net.num_layers)]
    for u, v in zip(a, b):
        np.testing.assert_array_equal(u.view(np.uint32), v.view(np.uint32))


def test_recurrent_driver_contract_tokens_and_perplexity():
    """Token input == one-hot input through the whole network; the perplexity figure follows recurrent.cc:239-247."""
    from nebula_amd import zoo
    from nebula_amd.net import Network
    print("CASE recurrent tokens + perplexity", flush=True)
    T, B, V, H = 6, 5, 40, 128
    rng = np.random.default_rng(31)
    cfg = zoo.lstm_cfg(batch=B, time_steps=T, input_size=V, hidden=H, layers=2, classes=V)
    onet = ob.OracleNet(cfg)
    blob = np.concatenate([rng.uniform(-1, 1, int(np.prod(sh))).astype(np.float32) / np.float32(np.sqrt(H))
                           for _, _, sh in ob.weight_layout(onet.specs)])
    onet.load_weights(blob)
    tokens = rng.integers(0, V, (T, B)).astype(np.uint32)
    labels = rng.integers(0, V, (T, B)).astype(np.uint32)
    x = np.zeros((T, B, V), np.float32)
    x[np.arange(T)[:, None], np.arange(B)[None, :], tokens] = 1.0
    ob.use_custom_gemm()
    want = onet.forward(x)
    probs_want = want[-1].reshape(T * B, V)
    with Network(cfg) as net:
        net.load_weight_blob(blob)
        net.set_input(x)
        net.forward()
        dense = [net.output(i) for i in range(net.num_layers)]
        net.set_input_tokens(tokens)
        net.forward()
        tok = [net.output(i) for i in range(net.num_layers)]
        for u, v in zip(dense, tok):
            np.testing.assert_array_equal(u.view(np.uint32), v.view(np.uint32))
        assert rel(tok[-1], probs_want.ravel()) <= TOL
        cum = 0.0
        for it in range(2):                      # two "iterations" of the driver on the same batch
            got = net.accumulate_perplexity(labels)
            cum = np.float32(cum + ob.target_prob_sum(probs_want, labels.ravel()))
            assert abs(got - ob.perplexity(float(cum), (it + 1) * T * B)) <= 1e-4 * got
        net.set_input(x)                          # back to the dense input
        net.forward()
        np.testing.assert_array_equal(net.output(0).view(np.uint32), dense[0].view(np.uint32))


@pytest.mark.parametrize("H,V", [(128, 40), (96, 37)])
def test_rnn_token_input_equals_one_hot_input(H, V):
    """rnn_large's shape in small: normalised [rnn] layers fed by the recurrent driver's one-hot rows.  Token input
    (a gather of input-gate weight columns) must equal the dense one-hot product bit for bit, for the one-launch
    step kernel (width 128) and the general path (width 96, odd vocabulary), and match the oracle."""
    from nebula_amd import zoo
    from nebula_amd.net import Network
    print("CASE rnn tokens", H, V, flush=True)
    T, B = 5, 6
    rng = np.random.default_rng(H + V)
    cfg = zoo.rnn_cfg(batch=B, time_steps=T, input_size=V, hidden=H, layers=2)
    onet = ob.OracleNet(cfg)
    blob = _random_weights(onet.specs, rng)
    onet.load_weights(blob)
    tokens = rng.integers(0, V, (T, B)).astype(np.uint32)
    x = np.zeros((T, B, V), np.float32)
    x[np.arange(T)[:, None], np.arange(B)[None, :], tokens] = 1.0
    ob.use_custom_gemm()
    want = onet.forward(x)
    with Network(cfg) as net:
        net.load_weight_blob(blob)
        net.set_input(x)
        net.forward()
        dense = [net.output(i) for i in range(net.num_layers)]
        net.set_input_tokens(tokens)
        net.forward()
        tok = [net.output(i) for i in range(net.num_layers)]
        for i, (u, v) in enumerate(zip(dense, tok)):
            np.testing.assert_array_equal(u.view(np.uint32), v.view(np.uint32), err_msg="layer %d" % i)
            assert rel(v, want[i].ravel()) <= TOL, (i, rel(v, want[i].ravel()))
        # a token outside the vocabulary is an all-zero input row
        tokens2 = tokens.copy(); tokens2[1, 2] = V + 3
        x2 = x.copy(); x2[1, 2, :] = 0.0
        net.set_input(x2)
        net.forward()
        d2 = net.output(0)
        net.set_input_tokens(tokens2)
        net.forward()
        np.testing.assert_array_equal(net.output(0).view(np.uint32), d2.view(np.uint32))


def test_image_driver_topk_count(golden_dir):
    """Running top-k match count of the image driver on the DBN fixture's probabilities."""
    from nebula_amd.net import Network
    print("CASE topk through network", flush=True)
    g = np.load(os.path.join(golden_dir, "dbn_small.npz"))
    with Network(str(g["cfg"])) as net:
        net.load_weight_blob(g["weights"])
        net.set_input(g["input"])
        net.forward()
        probs = g["out_03"].reshape(net.batch_size, -1)
        labels = np.array([0, 3, 1, 4], np.uint32)
        total = 0
        for k in (1, 2):
            total += ob.topk_matches(probs, labels, k)
            assert net.accumulate_topk(labels, k) == total


def test_in_place_shortcuts_on_golden_resnet(golden_dir):
    """shortcut_in_place=1 on the golden shortcut network: tensors that survive the pass equal the reference's, a tensor
    written over holds its writer's output, and shortcuts of another shape than their connection keep their own tensor."""
    from nebula_amd.net import Network
    g = np.load(os.path.join(golden_dir, "resnet_shortcuts.npz"))
    cfg = str(g["cfg"]).replace("[net]\n", "[net]\nfuse_shortcut=1\nshortcut_in_place=1\n", 1)
    with Network(cfg) as net:
        net.load_weight_blob(g["weights"])
        net.set_input(g["input"])
        net.forward()
        kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
        for i, k in enumerate(kinds):
            w = net.output_writer(i)
            if w == i:
                assert rel(net.output(i), g["out_%02d" % i]) <= TOL, (i, k)
            else:
                assert w > i
                if kinds[w] not in ("dropout_layer", "cost_layer"):
                    assert rel(net.output(i), g["out_%02d" % w]) <= TOL, (i, k, w)


def test_in_place_shortcut_is_refused_while_the_connection_is_still_read():
    """Two shortcuts add the same tensor.  The first must not write over it (the second still reads it); the second may."""
    from nebula_amd.net import Network
    print("CASE in-place liveness", flush=True)
    body = ("\n[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=relu\n"          # 0: the shared connection
            "\n[convolutional]\nfilters=16\nsize=1\nstride=1\npadding=0\nactivation=relu\n"          # 1
            "\n[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=linear\n"        # 2 (fused with 3)
            "\n[shortcut]\nhops=3\nactivation=relu\n"                                                 # 3: adds layer 0
            "\n[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=linear\n"        # 4 (fused with 5)
            "\n[shortcut]\nhops=5\nactivation=relu\n"                                                 # 5: adds layer 0 again
            "\n[avgpool]\nsize=12\nstride=12\npadding=0\n\n[connected]\noutput=10\nactivation=linear\n\n[softmax]\ngroups=1\n")
    head = "[net]\nbatch=3\nheight=12\nwidth=12\nchannels=4\nconv_split=0\n%s"
    rng = np.random.default_rng(23)
    onet = ob.OracleNet(head % "" + body)
    blob = _random_weights(onet.specs, rng)
    x = rng.standard_normal((3, 4, 12, 12)).astype(np.float32)
    onet.load_weights(blob)
    ob.use_custom_gemm()
    want = onet.forward(x)
    with Network(head % "fuse_shortcut=1\nshortcut_in_place=1\n" + body) as net:
        net.load_weight_blob(blob)
        net.set_input(x)
        net.forward()
        assert net.output_writer(3) == 3          # kept its own tensor: layer 5 still needs layer 0
        assert net.output_writer(0) == 5          # the last reader wrote over it
        for i in (1, 3, 5, 6, 7, 8):
            assert rel(net.output(i), want[i].ravel()) <= TOL, i
        np.testing.assert_array_equal(net.output(0).view(np.uint32), net.output(5).view(np.uint32))
