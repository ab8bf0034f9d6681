#!/usr/bin/env python3
"""Writes the golden vectors in this directory from the compiled, unmodified reference.

Runs only where /root/reference exists (the authoring container): it builds
oracle/_ref/libnebula_ref.so from the reference's own sources (oracle/Makefile, target `ref`,
CUSTOM_BLAS build = the reference's hand-written GEMM) and records, for a handful of small
networks, the input, the .wgh weight blob and the output of every layer (plus the maxpool
argmax tables).  The .npz files hold data only; the reference itself never travels.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as ob  # noqa: E402

CASES = {}

CASES["convnet_mixed"] = ("""
[net]
batch=2
height=13
width=12
channels=3
num_threads=2

[convolutional]
batch_normalize=1
filters=6
size=3
stride=1
padding=1
activation=leaky

[maxpool]
size=3
stride=2

[convolutional]
filters=8
size=3
stride=2
padding=0
activation=relu

[avgpool]
size=2
stride=1
padding=1

[connected]
batch_normalize=1
output=9
activation=logistic

[dropout]
probability=0.5

[connected]
output=7
activation=linear

[softmax]

[cost]
type=l2
""", "uniform")

CASES["alexnet_conv1_small"] = ("""
[net]
batch=3
height=35
width=35
channels=3

[convolutional]
filters=16
size=11
stride=4
padding=0
activation=relu

[maxpool]
size=3
stride=2
padding=0
""", "uniform")

# Bottleneck with channel growth (4 -> 16, only the first 4 channels get the residual), then a
# stride-2 entry block (conn is subsampled [::2, ::2]) and a 19 -> 10 style odd size where the
# integer division gives stride 1.
CASES["resnet_shortcuts"] = ("""
[net]
batch=2
height=19
width=19
channels=3
num_threads=3

[convolutional]
batch_normalize=1
filters=4
size=7
stride=2
padding=3
activation=relu

[maxpool]
size=3
stride=2
padding=0

[convolutional]
batch_normalize=1
filters=4
size=1
stride=1
padding=0
activation=relu

[convolutional]
batch_normalize=1
filters=4
size=3
stride=1
padding=1
activation=relu

[convolutional]
batch_normalize=1
filters=16
size=1
stride=1
padding=0
activation=linear

[shortcut]
hops=4
activation=relu

[convolutional]
batch_normalize=1
filters=8
size=1
stride=1
padding=0
activation=leaky

[convolutional]
batch_normalize=1
filters=8
size=3
stride=2
padding=1
activation=leaky

[convolutional]
batch_normalize=1
filters=32
size=1
stride=1
padding=0
activation=linear

[shortcut]
hops=4
activation=leaky

[avgpool]
size=2
stride=2
padding=0

[connected]
output=5
activation=linear

[softmax]
""", "normal")

CASES["lstm_plain"] = ("""
[net]
batch=2
input_size=5
time_steps=3
num_threads=2

[lstm]
output=4
activation=linear

[lstm]
output=6
activation=linear

[connected]
output=7
activation=linear

[softmax]
""", "normal")

# The shipped lstm cfgs set batch_normalize=1 on the [lstm] section (benchmarks/lstm_large/network.cfg)
# and the section's activation is applied inside every sub-layer.
CASES["lstm_bn_tanh"] = ("""
[net]
batch=3
input_size=6
time_steps=4

[lstm]
batch_normalize=1
output=5
activation=tanh

[connected]
batch_normalized=1
output=4
activation=linear

[softmax]
groups=1
""", "normal")

# rnn_layer.cc: three connected sub-layers per [rnn]; step 0 takes its hidden and output gates' inputs from
# the neighbouring sub-layer instead of the running state.
CASES["rnn_plain"] = ("""
[net]
batch=3
input_size=7
time_steps=4

[rnn]
output=6
activation=relu

[rnn]
output=5
activation=linear

[connected]
output=8
activation=linear

[softmax]
""", "normal")

# The shipped rnn cfgs (benchmarks/rnn_large/network.cfg) normalize every sub-layer.
CASES["rnn_bn_leaky"] = ("""
[net]
batch=2
input_size=9
time_steps=5

[rnn]
batch_normalize=1
output=7
activation=leaky

[connected]
output=6
activation=linear

[softmax]
""", "normal")

# benchmarks/dbn_*/network.cfg: [rbm] layers run as connected layers without batchnorm at inference.
CASES["dbn_small"] = ("""
[net]
batch=4
height=6
width=5
channels=3

[rbm]
output=20
k_step=1
activation=logistic

[rbm]
output=9
k_step=1
activation=logistic

[connected]
output=5
activation=linear

[softmax]
""", "uniform")

# Seeds of the fixtures already committed stay what they were; new cases get their own.
SEEDS = {"alexnet_conv1_small": 1000, "convnet_mixed": 1001, "lstm_bn_tanh": 1002, "lstm_plain": 1003,
         "resnet_shortcuts": 1004, "rnn_plain": 2007, "rnn_bn_leaky": 2006, "dbn_small": 2005}


def make_weights(specs, rng):
    parts = []
    for li, name, shape in ob.weight_layout(specs):
        base = name.split(".")[-1]
        if base == "weight":
            fan_in = int(np.prod(shape[1:]))
            a = rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)
        elif base == "bias":
            a = rng.standard_normal(shape) * 0.1
        elif base == "scale":
            a = rng.uniform(0.8, 1.2, shape)
        elif base == "mean":
            a = rng.standard_normal(shape) * 0.1
        elif base == "var":
            a = rng.uniform(0.5, 1.5, shape)
        parts.append(a.astype(np.float32).ravel())
    return np.concatenate(parts) if parts else np.zeros(0, np.float32)


def main():
    if ob.ref() is None:
        sys.exit("the reference tree is not present: golden vectors can only be written in the authoring container")
    only = set(sys.argv[1:])       # optional: names of the cases to (re)write
    for name, (cfg, dist) in sorted(CASES.items()):
        if only and name not in only:
            continue
        rng = np.random.default_rng(SEEDS[name])
        net, specs = ob.plan_network(cfg)
        rn = ob.RefNet(cfg)
        n_in = rn.input_size * rn.batch_size
        x = (rng.random(n_in) if dist == "uniform" else rng.standard_normal(n_in)).astype(np.float32)
        blob = make_weights(specs, rng)
        rn.load_weights(blob)
        outs = rn.forward(x)
        data = {"cfg": np.array(cfg), "input": x, "weights": blob,
                "batch_size": np.array(rn.batch_size), "time_step": np.array(rn.time_step)}
        for i, o in enumerate(outs):
            d = rn.layer_dims(i)
            data["out_%02d" % i] = o
            data["dims_%02d" % i] = np.array([d["output_channel"], d["output_height"], d["output_width"],
                                              d["output_size"], d["layer_type"], d["activation_type"]], np.uint32)
            idx = rn.pool_index(i)
            if idx is not None:
                data["idx_%02d" % i] = idx
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **data)
        print("%-22s layers=%2d  %6.1f KB" % (name, len(outs), os.path.getsize(path) / 1024))

    if only and "activations" not in only:
        return
    # all 13 activations on a fixed vector with the awkward points in it
    rng = np.random.default_rng(77)
    x = (rng.standard_normal(4096) * 3).astype(np.float32)
    x[:24] = [0, -0.0, 1, -1, 4, -4, 4.0001, -4.0001, 0.5, -0.5, 2, 3, -2, -3, 1e-30, -1e-30, 88, -88, 1.5, 2.5,
              7.9, -7.9, 1e-8, 100.0]
    data = {"input": x}
    for name in ob.ACT_NAMES[1:]:
        y = x.copy()
        assert ob.ref().ref_activation(ob.ACT[name], ob._fp(y), y.size) == 0
        data[name] = y
    path = os.path.join(HERE, "activations.npz")
    np.savez_compressed(path, **data)
    print("%-22s %6.1f KB" % ("activations", os.path.getsize(path) / 1024))


if __name__ == "__main__":
    main()
