"""The C++ layer framework without a GPU (dry-run networks, device = -1): cfg parsing quirks, shape
inference, the .wgh field order and the error behaviour, checked against the reference's own numbers
(golden fixtures hold every layer's dims as the compiled reference reported them) and the oracle's planner."""
import glob
import os

import numpy as np
import pytest

from nebula_amd import zoo
from nebula_amd.net import Network, NetworkError
from oracle import binding as ob

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
NETS = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "*.npz")) if not p.endswith("activations.npz"))


def dry(cfg, **kw):
    return Network(cfg, device=-1, **kw)


@pytest.mark.parametrize("name", NETS)
def test_layer_dims_match_reference_fixture(name):
    g = np.load(os.path.join(GOLDEN, name + ".npz"))
    with dry(str(g["cfg"])) as net:
        assert net.batch_size == int(g["batch_size"]) and net.time_step == int(g["time_step"])
        for i in range(net.num_layers):
            info, dims = net.layer_info(i), g["dims_%02d" % i]
            assert info["output_size"] == dims[3] and info["layer_type"] == dims[4] and info["activation_type"] == dims[5]
            if info["kind"] in ("convolutional_layer", "maxpool_layer", "avgpool_layer", "shortcut_layer"):
                assert (info["output_channel"], info["output_height"], info["output_width"]) == tuple(dims[:3])
        # the .wgh blob the reference consumed has exactly the size our field table adds up to
        assert sum(f[2] for f in net.weight_layout()) == g["weights"].size
        net.load_weight_blob(g["weights"])


@pytest.mark.parametrize("name", sorted(zoo.WORKLOADS))
def test_zoo_shapes_and_weight_layout_match_oracle_planner(name):
    cfg = zoo.WORKLOADS[name](2)
    _, specs = ob.plan_network(cfg)
    with dry(cfg) as net:
        assert net.num_layers == len(specs)
        for i, sp in enumerate(specs):
            info = net.layer_info(i)
            if sp.kind in ("convolutional", "maxpool", "avgpool"):
                assert (info["output_channel"], info["output_height"], info["output_width"]) == sp.out, (name, i)
            assert info["output_size"] == sp.out_size, (name, i, sp.kind)
        ours = [(li, kind, count) for li, kind, count, _ in net.weight_layout()]
        theirs = [(li, n.split(".")[-1], int(np.prod(sh))) for li, n, sh in ob.weight_layout(specs)]
        assert ours == theirs


def test_resnet50_flop_count():
    with dry(zoo.resnet50_cfg(64)) as net:
        flop = sum(net.layer_flop(i) for i in range(net.num_layers))
        assert abs(flop / 1e9 - 7.459) < 0.01     # GFLOP per image, 49 convs + FC


def test_cfg_quirks():
    cfg = ("[net]\nBATCH = 2\nheight=5\nwidth = 5\nchannels=2\nbogus=1\n# comment\n\n[convolutional]\n"
           "FILTERS=3\nsize = 3\nSTRIDE=1\npadding=1\nACTIVATION=ReLU\nfilters=9\nbatch_normalized=1\n")
    with dry(cfg) as net:
        info = net.layer_info(0)
        assert (info["output_channel"], info["output_height"], info["output_width"]) == (3, 5, 5)   # first filters= wins
        assert info["activation_type"] == ob.ACT["relu"]
        assert [f[1] for f in net.weight_layout()] == ["bias", "weight"]      # the misspelt batch_normalized is ignored
    with dry("[net]\nbatch=3\ninput_size=7\ntime_steps=4\n[lstm]\noutput=5\nactivation=linear\n[softmax]\n") as net:
        assert (net.batch_size, net.time_step, net.input_size) == (12, 4, 7)     # batch *= time_steps


def test_pool_defaults_and_size_rule():
    with dry("[net]\nbatch=1\nheight=12\nwidth=12\nchannels=1\n[maxpool]\nsize=3\nstride=2\n") as net:
        info = net.layer_info(0)           # default padding (3-1)/2 = 1 -> (12 + 2) / 2 = 7
        assert (info["padding"], info["output_height"]) == (1, 7)
    with dry("[net]\nbatch=1\nheight=8\nwidth=8\nchannels=1\n[avgpool]\nstride=2\n") as net:
        assert net.layer_info(0)["output_height"] == 4    # window defaults to the stride, padding to 0


def test_errors():
    with pytest.raises(NetworkError, match="unknown layer type"):
        dry("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[bogus]\nx=1\n")
    with pytest.raises(NetworkError, match="undefined activation type"):
        dry("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[convolutional]\nfilters=2\nsize=3\nactivation=swish\n")
    with pytest.raises(NetworkError, match="undefined activation type"):
        dry("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[connected]\noutput=2\n")          # no activation= at all
    with pytest.raises(NetworkError, match="invalid config"):
        dry("[net]\nbatch=1\nheight\n")
    with pytest.raises(NetworkError, match="failed to open"):
        dry("/nonexistent/network.cfg", is_text=False)
    with pytest.raises(NetworkError, match="hops"):
        dry("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[convolutional]\nfilters=2\nsize=1\nactivation=linear\n"
            "[shortcut]\nhops=5\nactivation=linear\n")
    with pytest.raises(NetworkError, match="geometry"):
        dry("[net]\nbatch=1\nheight=2\nwidth=2\nchannels=1\n[convolutional]\nfilters=2\nsize=5\nactivation=linear\n")
    with dry("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[connected]\noutput=3\nactivation=linear\n") as net:
        with pytest.raises(NetworkError, match="no device"):
            net.forward()
        with pytest.raises(NetworkError, match="shorter"):
            net.load_weight_blob(np.zeros(5, np.float32))


def test_weights_round_trip_without_device(tmp_path):
    from nebula_amd import net as netmod
    g = np.load(os.path.join(GOLDEN, "lstm_bn_tanh.npz"))
    with dry(str(g["cfg"])) as net:
        net.load_weight_blob(g["weights"])
        out = str(tmp_path / "out.wgh")
        assert netmod.lib().nbl_net_store_weights(net.h, out.encode()) == 0
        np.testing.assert_array_equal(np.fromfile(out, np.float32), g["weights"])


def test_tensor_ownership_of_fused_and_in_place_shortcuts():
    """Which layer's values a layer's output holds after a pass, decided at build time (no device needed): a fused
    convolution shares its shortcut's tensor; with shortcut_in_place=1 a same-shape shortcut writes over its connection's
    tensor unless a later layer still reads that tensor; a fusion is skipped while the convolution's own output is read."""
    from nebula_amd.net import Network
    from nebula_amd import zoo
    conv = "\n[convolutional]\nfilters=16\nsize=3\nstride=1\npadding=1\nactivation=%s\n"
    body = (conv % "relu" + conv % "relu" + conv % "linear" + "\n[shortcut]\nhops=3\nactivation=relu\n"      # 3 adds layer 0
            + conv % "linear" + "\n[shortcut]\nhops=5\nactivation=relu\n"                                   # 5 adds layer 0 again
            + "\n[avgpool]\nsize=12\nstride=12\npadding=0\n\n[connected]\noutput=10\nactivation=linear\n\n[softmax]\ngroups=1\n")
    head = "[net]\nbatch=3\nheight=12\nwidth=12\nchannels=4\n%s"
    writers = lambda cfg: [(lambda n: [n.output_writer(i) for i in range(n.num_layers)])(Network(cfg, device=-1))][0]
    assert writers(head % "" + body) == list(range(9))
    assert writers(head % "fuse_shortcut=1\n" + body) == [0, 1, 3, 3, 5, 5, 6, 7, 8]
    # shortcut 3 keeps its tensor (layer 5 still reads layer 0), shortcut 5 takes layer 0's
    assert writers(head % "fuse_shortcut=1\nshortcut_in_place=1\n" + body) == [5, 1, 3, 3, 5, 5, 6, 7, 8]
    # in place needs the fusion
    assert writers(head % "shortcut_in_place=1\n" + body) == list(range(9))
    # shortcut 4 (hops=3) adds the output of convolution 1, so the pair (1, 2) cannot be fused: the sum would replace what
    # shortcut 4 needs.  Shortcut 4 itself is fused with convolution 3 and may write over layer 1's tensor: its only other
    # reader, shortcut 2, runs earlier.
    twice = (conv % "relu" + conv % "linear" + "\n[shortcut]\nhops=2\nactivation=relu\n" + conv % "linear"
             + "\n[shortcut]\nhops=3\nactivation=linear\n\n[softmax]\ngroups=1\n")
    w = writers(head % "fuse_shortcut=1\nshortcut_in_place=1\n" + twice)
    assert w == [0, 4, 2, 4, 4, 5], w
    assert writers(head % "fuse_shortcut=1\n" + twice) == [0, 1, 2, 4, 4, 5]
    # ResNet-50: sixteen fused convolutions; in place, every stage shares one tensor from its first block's output on
    kinds = lambda n: [n.layer_info(i)["kind"] for i in range(n.num_layers)]
    net = Network(zoo.resnet50_cfg(2, fuse_shortcut=True), device=-1)
    own = [i for i, k in enumerate(kinds(net)) if k not in ("cost_layer", "dropout_layer")]
    assert sum(net.output_writer(i) != i for i in own) == 16
    cost = net.num_layers - 1          # the closing [cost] layer has no tensor: it reports its producer, the softmax layer
    assert kinds(net)[cost] == "cost_layer" and net.output_writer(cost) == cost - 1
    net = Network(zoo.resnet50_cfg(2, fuse_shortcut=True, in_place=True), device=-1)
    sc = [i for i, k in enumerate(kinds(net)) if k == "shortcut_layer"]
    assert [net.output_writer(i) for i in sc] == [13, 13, 13, 29, 29, 29, 29, 53, 53, 53, 53, 53, 53, 65, 65, 65]


def test_carry_state_key_and_calls_on_a_dry_run_network():
    """[net] carry_state=1 is parsed for recurrent nets; the state calls are harmless before weights exist and on
    networks without [lstm] layers."""
    cfg = zoo.lstm_cfg(batch=2, time_steps=3, input_size=8, hidden=16, layers=2, classes=5)
    for text in (cfg, cfg.replace("[net]\n", "[net]\ncarry_state=1\n", 1), zoo.alexnet_cfg(1)):
        with dry(text) as net:
            net.set_carry_state(True)
            net.reset_state()
            net.set_carry_state(False)
