"""Measures the convolution launches of the shipped networks on the device and writes the launch table.

    python -m nebula_amd.tune [--out nebula_amd/launch_tables/gfx950.txt] [--rounds 3] [--workloads resnet50,vgg16,...] [--merge]

Every round empties the in-memory table, builds each network at the batch size it is benchmarked at and runs one
forward pass, which measures every convolution problem the table does not hold (nbl_conv2d_fwd's tile search) and
enters the winner.  A problem's final entry is the choice most rounds agreed on (ties: the one with the lowest
measured time), so a single noisy search does not decide a layer.  The file it writes is what libnebula_hip.so
reads on first use; a network of one's own is added by running it once and calling nbl_launch_table_save.
--merge keeps every entry the output file already holds and adds only problems it does not list (the benchmarked
networks' entries, which the committed profiles were taken with, then stay as they are).
"""
import argparse
import collections
import os
import sys
import tempfile

import numpy as np

from . import hip, zoo
from .net import Network

HEADER = """# gfx950 (MI355X) convolution launch table: tile shape and k slices per problem, measured on the device by
# `python -m nebula_amd.tune` (%s).
# conv C H W F k stride pad batch res_c res_h res_w in_place tile slices us
"""

# (name, cfg text builder, input distribution, weight distribution)
WORKLOADS = collections.OrderedDict([
    ("conv1", (lambda: zoo.conv1_pool_cfg(32), "he")),
    ("alexnet", (lambda: zoo.alexnet_cfg(128), "he")),
    ("vgg16", (lambda: zoo.vgg16_cfg(32), "he")),
    ("resnet50", (lambda: zoo.resnet50_cfg(64, fuse_shortcut=True, in_place=True), "he")),
    ("resnet50_fused", (lambda: zoo.resnet50_cfg(64, fuse_shortcut=True), "he")),
    ("resnet50_plain", (lambda: zoo.resnet50_cfg(64), "he")),
])
# the same networks at other batch sizes (not benchmarked; listed so that a first pass at these sizes measures nothing)
for _b in (16, 32, 128, 256):
    WORKLOADS["resnet50_b%d" % _b] = ((lambda b=_b: zoo.resnet50_cfg(b, fuse_shortcut=True, in_place=True)), "he")
for _b in (16, 64, 128):
    WORKLOADS["vgg16_b%d" % _b] = ((lambda b=_b: zoo.vgg16_cfg(b)), "he")
for _b in (32, 64, 256, 512):
    WORKLOADS["alexnet_b%d" % _b] = ((lambda b=_b: zoo.alexnet_cfg(b)), "he")
BENCHMARKED = ["conv1", "alexnet", "vgg16", "resnet50", "resnet50_fused", "resnet50_plain"]


def read_table(path):
    """{key tuple of 12 ints: (tile, slices, us)}"""
    out = {}
    for line in open(path):
        line = line.split("#", 1)[0].split()
        if not line:
            continue
        assert line[0] == "conv" and len(line) >= 15, line
        out[tuple(int(v) for v in line[1:13])] = (line[13], int(line[14]), float(line[15]) if len(line) > 15 else 0.0)
    return out


def write_table(path, entries, note):
    with open(path, "w") as f:
        f.write(HEADER % note)
        for key in sorted(entries):
            tile, slices, us = entries[key]
            f.write("conv %s %s %d %.1f\n" % (" ".join(str(v) for v in key), tile, slices, us))


def measure_round(names, log):
    l = hip.lib()
    l.nbl_launch_table_clear()
    l.nbl_launch_table_set_search(1)
    rng = np.random.default_rng(20240611)
    for name in names:
        cfg_fn, wdist = WORKLOADS[name]
        with Network(cfg_fn()) as net:
            net.load_weight_blob(zoo.synthetic_weights(net.weight_layout(), rng, wdist))
            n_in = net.batch_size * net.input_size
            net.set_input(rng.standard_normal(n_in).astype(np.float32))
            net.forward()
            net.sync()
        log("  %s: table holds %d problems" % (name, l.nbl_launch_table_size()))
    with tempfile.NamedTemporaryFile("w", suffix=".txt", delete=False) as f:
        path = f.name
    try:
        if l.nbl_launch_table_save(path.encode()) < 0:
            raise RuntimeError(l.nbl_last_error(None).decode())
        return read_table(path)
    finally:
        os.unlink(path)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(hip.PKG, "launch_tables", "gfx950.txt"))
    ap.add_argument("--rounds", type=int, default=3)
    ap.add_argument("--workloads", default=",".join(BENCHMARKED), help="any of: " + ", ".join(WORKLOADS))
    ap.add_argument("--merge", action="store_true", help="keep the entries the output file already holds; add new problems only")
    args = ap.parse_args()
    names = [n for n in args.workloads.split(",") if n]
    log = lambda *a: print(*a, file=sys.stderr, flush=True)
    votes = collections.defaultdict(list)
    for r in range(args.rounds):
        log("round %d of %d" % (r + 1, args.rounds))
        for key, choice in measure_round(names, log).items():
            votes[key].append(choice)
    entries = {}
    for key, seen in votes.items():
        count = collections.Counter((t, s) for t, s, _ in seen)
        best_n = max(count.values())
        tied = [c for c, n in count.items() if n == best_n]
        pick = min(tied, key=lambda c: min(us for t, s, us in seen if (t, s) == c))
        entries[key] = (pick[0], pick[1], min(us for t, s, us in seen if (t, s) == pick))
    note = "%d rounds over %s" % (args.rounds, ", ".join(names))
    if args.merge and os.path.exists(args.out):
        kept = read_table(args.out)
        log("kept %d problems of %s, %d new" % (len(kept), args.out, len(set(entries) - set(kept))))
        entries.update(kept)
        note = "benchmarked networks first; then, merged, " + note
    os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
    write_table(args.out, entries, note)
    log("wrote %d problems to %s" % (len(entries), args.out))


if __name__ == "__main__":
    main()
