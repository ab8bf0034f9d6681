"""The generated cfgs reproduce the reference's shipped topologies (checked against the reference's
own cfg files where that tree exists) and chain to the published shapes."""
import os

import pytest

from nebula_amd import zoo
from oracle import binding as ob

REF = "/root/reference/benchmarks"


def skeleton(cfg_text):
    out = []
    for name, kv in ob.parse_cfg(cfg_text)[1:]:
        keys = ("filters", "size", "stride", "padding", "hops", "output", "batch_normalize")
        out.append((name,) + tuple((k, kv[k]) for k in keys if k in kv))
    return out


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not present")
@pytest.mark.parametrize("ours,theirs", [("alexnet", "alexnet_large"), ("vgg16", "vgg_large"), ("resnet50", "resnet_large")])
def test_same_layer_sequence_as_shipped_cfg(ours, theirs):
    ref = open(os.path.join(REF, theirs, "network.cfg")).read()
    assert skeleton(zoo.WORKLOADS[ours]()) == skeleton(ref)


def test_resnet50_shapes_and_flops():
    net, specs = ob.plan_network(zoo.resnet50_cfg(64))
    convs = [s for s in specs if s.kind == "convolutional"]
    assert len(convs) == 49 and sum(s.kind == "shortcut" for s in specs) == 16
    assert specs[0].out == (64, 112, 112) and specs[1].out == (64, 56, 56)
    avg = [s for s in specs if s.kind == "avgpool"][0]
    assert (avg.C, avg.H, avg.W) == (2048, 7, 7) and avg.out == (2048, 1, 1)
    flop = sum(2.0 * s.F * s.out[1] * s.out[2] * s.C * s.k * s.k for s in convs)
    fc = [s for s in specs if s.kind == "connected"][0]
    flop += 2.0 * fc.I * fc.O
    assert abs(flop / 1e9 - 7.459) < 0.01            # GFLOP per image


def test_alexnet_vgg_lstm_shapes():
    _, a = ob.plan_network(zoo.alexnet_cfg())
    assert [s.out for s in a if s.kind == "maxpool"] == [(96, 27, 27), (256, 13, 13), (256, 6, 6)]
    assert [s.I for s in a if s.kind == "connected"] == [9216, 4096, 4096]
    _, v = ob.plan_network(zoo.vgg16_cfg())
    assert [s.out[1] for s in v if s.kind == "maxpool"] == [112, 56, 28, 14, 7]
    assert [s.I for s in v if s.kind == "connected"][0] == 25088
    net, l = ob.plan_network(zoo.lstm_cfg())
    assert net["recurrent"] and net["time_steps"] == 64 and [s.kind for s in l[:2]] == ["lstm", "lstm"]
    _, c = ob.plan_network(zoo.conv1_pool_cfg())
    assert c[0].out == (96, 55, 55) and c[1].out == (96, 27, 27)
