"""Recorded forward passes (HIP graph, [net] key hip_graph / nbl_net_set_graph): every replay must equal the
eager pass of the same network on the same input bit for bit, on several replays with eager work of the
program in between, and anything that changes what a pass launches must start the recording over."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402
from test_gpu_networks import MINI_RESNET, _random_weights  # noqa: E402


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def all_outputs(net):
    return [net.output(i).copy() for i in range(net.num_layers)]


def small_recurrent(kind, last_step_only=False):
    from nebula_amd import zoo
    if kind == "lstm":
        return zoo.lstm_cfg(batch=8, time_steps=5, input_size=96, hidden=64, layers=2, classes=50,
                            last_step_only=last_step_only), (5, 8, 96)
    return zoo.rnn_cfg(batch=8, time_steps=5, input_size=96, hidden=64, layers=3, last_step_only=last_step_only), (5, 8, 96)


CASES = ["mini_resnet", "mini_resnet_fused", "mini_resnet_fused_in_place", "lstm", "lstm_last_step", "rnn", "dbn_like"]


def build_case(name, rng):
    if name.startswith("mini_resnet"):
        keys = "fuse_shortcut=1\nshortcut_in_place=1\n" if name.endswith("in_place") else "fuse_shortcut=1\n" if name.endswith("fused") else ""
        cfg = MINI_RESNET.replace("[net]\n", "[net]\n" + keys, 1)
        shape = (4, 3, 32, 32)
    elif name.startswith("lstm"):
        cfg, shape = small_recurrent("lstm", name.endswith("last_step"))
    elif name == "rnn":
        cfg, shape = small_recurrent("rnn")
    else:
        cfg = ("[net]\nbatch=6\nheight=1\nwidth=1\nchannels=200\n[rbm]\noutput=96\nactivation=logistic\n"
               "[rbm]\noutput=64\nactivation=logistic\n[connected]\noutput=10\nactivation=linear\n[softmax]\n")
        shape = (6, 200, 1, 1)
    specs = ob.OracleNet(cfg).specs
    blobs = [_random_weights(specs, rng) for _ in range(2)]
    xs = [rng.standard_normal(shape).astype(np.float32) for _ in range(3)]
    return cfg, blobs, xs


@pytest.mark.parametrize("name", CASES)
def test_replays_equal_eager_passes(name):
    from nebula_amd.net import Network
    print("CASE graph replay", name, flush=True)
    rng = np.random.default_rng(len(name) * 7 + 1)
    cfg, blobs, xs = build_case(name, rng)
    with Network(cfg) as net, Network(cfg) as other:
        net.load_weight_blob(blobs[0])
        other.load_weight_blob(blobs[1])
        # eager results of this very network (same tile choices as the recorded pass will have)
        want = []
        for x in xs:
            net.set_input(x)
            net.forward()
            want.append(all_outputs(net))
        assert not net.graph_active
        net.set_graph(True)
        order = [0, 0, 1, 2, 0, 1]           # pass 1 eager, pass 2 recorded, then replays
        for n, which in enumerate(order):
            net.set_input(xs[which])
            net.forward()
            assert net.graph_active == (n >= 1), (n, net.graph_active)
            got = all_outputs(net)
            for i, (g, w) in enumerate(zip(got, want[which])):
                np.testing.assert_array_equal(bits(g), bits(w), err_msg="%s pass %d layer %d" % (name, n, i))
            # eager work of the program between the replays, on another network of the same context kind
            other.set_input(xs[(which + 1) % 3])
            other.forward()
            other.sync()
        # new weights: the recorded pass is dropped, the next ones are eager, recorded, replayed
        net.load_weight_blob(blobs[1])
        assert not net.graph_active
        for n in range(3):
            net.set_input(xs[1])
            net.forward()
            assert net.graph_active == (n >= 1)
            got = all_outputs(net)
        other.set_input(xs[1])
        other.forward()
        # `other` holds the same weights; its tile search may differ, so compare within the layer tolerance
        for i, (g, w) in enumerate(zip(got, all_outputs(other))):
            scale = max(float(np.abs(w).max()), 1e-30)
            assert float(np.abs(g.astype(np.float64) - w.astype(np.float64)).max()) / scale <= 1e-4, (name, i)
        # switching the recording off returns to eager passes with the same results
        net.set_graph(False)
        net.set_input(xs[1])
        net.forward()
        assert not net.graph_active
        for i, (g, w) in enumerate(zip(all_outputs(net), got)):
            np.testing.assert_array_equal(bits(g), bits(w), err_msg="%s eager after graph, layer %d" % (name, i))


def test_token_input_and_softmax_copy_start_the_recording_over():
    from nebula_amd.net import Network
    print("CASE graph invalidation", flush=True)
    rng = np.random.default_rng(5)
    cfg, shape = small_recurrent("lstm")
    T, B, V = shape
    specs = ob.OracleNet(cfg).specs
    blob = _random_weights(specs, rng)
    tokens = rng.integers(0, V, size=(T, B)).astype(np.uint32)
    onehot = np.zeros(shape, np.float32)
    onehot.reshape(T * B, V)[np.arange(T * B), tokens.ravel()] = 1.0
    with Network(cfg) as net:
        net.load_weight_blob(blob)
        net.set_input(onehot)
        net.forward()
        dense = all_outputs(net)
        net.set_input_tokens(tokens)
        net.forward()
        gathered = all_outputs(net)
        net.set_graph(True)
        for mode, want in (("dense", dense), ("tokens", gathered), ("dense", dense)):
            for n in range(3):
                if mode == "dense":
                    net.set_input(onehot)
                else:
                    net.set_input_tokens(tokens)
                net.forward()
                assert net.graph_active == (n >= 1), (mode, n)
                for i, (g, w) in enumerate(zip(all_outputs(net), want)):
                    np.testing.assert_array_equal(bits(g), bits(w), err_msg="%s pass %d layer %d" % (mode, n, i))
        net.softmax_copy(False)
        for n in range(3):
            net.forward()
            assert net.graph_active == (n >= 1)
        for i, (g, w) in enumerate(zip(all_outputs(net), dense)):
            np.testing.assert_array_equal(bits(g), bits(w))
