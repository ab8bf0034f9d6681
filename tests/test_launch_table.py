"""The convolution launch table without a GPU: the file format (load / save / clear, malformed lines), and that the
table shipped with the library lists every convolution problem of the benchmarked networks at their benchmarked
batch sizes, so that none of them is ever searched (a forward pass is then a fixed sequence of launches, as the
reference's is: models/networks/network.cc:57-63)."""
import os

import pytest

from nebula_amd import hip, tune, zoo
from nebula_amd.net import Network

TABLE = os.path.join(hip.PKG, "launch_tables", "gfx950.txt")


@pytest.fixture(autouse=True)
def restore_table():
    yield
    hip.lib().nbl_launch_table_load(None)       # other tests in this process see the shipped table again
    hip.lib().nbl_launch_table_set_search(1)


def test_shipped_table_loads_and_round_trips(tmp_path):
    l = hip.lib()
    n = l.nbl_launch_table_load(None)
    assert n > 0, l.nbl_last_error(None).decode()
    assert l.nbl_launch_table_size() == n == len(tune.read_table(TABLE))
    out = str(tmp_path / "copy.txt")
    assert l.nbl_launch_table_save(out.encode()) == n
    mine, theirs = tune.read_table(out), tune.read_table(TABLE)
    assert {k: v[:2] for k, v in mine.items()} == {k: v[:2] for k, v in theirs.items()}
    assert l.nbl_launch_table_clear() == 0 and l.nbl_launch_table_size() == 0
    assert l.nbl_launch_table_load(out.encode()) == n


def test_every_entry_names_a_tile_shape_and_a_legal_slice_count():
    l = hip.lib()
    names = {l.nbl_conv2d_variant_name(v).decode() for v in range(l.nbl_conv2d_num_variants() + 1)}
    for key, (tile, slices, us) in tune.read_table(TABLE).items():
        assert tile in names and (slices == 0 or 2 <= slices <= 8), (key, tile, slices)
        if tile == "strip":
            assert key[0] <= 4 and key[8:] == (0, 0, 0, 0) and slices == 0       # few channels, no fused shortcut, never split
        if key[11]:
            assert key[8:11] == (key[3], (key[1] + 2 * key[6] - key[4]) // key[5] + 1, (key[2] + 2 * key[6] - key[4]) // key[5] + 1)


@pytest.mark.parametrize("bad", ["conv 1 2 3\n", "conv 3 8 8 4 3 1 1 2 0 0 0 0 nosuchtile 0 1.0\n",
                                 "conv 3 8 8 4 3 1 1 2 0 0 0 0 64x64 1 1.0\n", "conv 3 8 8 4 3 1 1 2 0 0 0 0 64x64 9\n", "pool 1 2\n"])
def test_malformed_file_is_refused_with_its_line_number(tmp_path, bad):
    l = hip.lib()
    before = l.nbl_launch_table_size()
    path = tmp_path / "bad.txt"
    path.write_text("# a comment\nconv 3 8 8 4 3 1 1 2 0 0 0 0 64x64 0 1.0   # fine\n\n" + bad)
    assert l.nbl_launch_table_load(str(path).encode()) < 0
    assert "line 4" in l.nbl_last_error(None).decode()
    assert l.nbl_launch_table_size() == before          # a refused file leaves the table as it was
    assert l.nbl_launch_table_load(str(tmp_path / "missing.txt").encode()) < 0
    assert "cannot open" in l.nbl_last_error(None).decode()


WORKLOADS = {"conv1": lambda: zoo.conv1_pool_cfg(32), "alexnet": lambda: zoo.alexnet_cfg(128), "vgg16": lambda: zoo.vgg16_cfg(32),
             "resnet50 (benchmarked: fused shortcuts written in place)": lambda: zoo.resnet50_cfg(64, fuse_shortcut=True, in_place=True),
             "resnet50 (fused)": lambda: zoo.resnet50_cfg(64, fuse_shortcut=True),
             "resnet50 (as the reference's cfg reads)": lambda: zoo.resnet50_cfg(64),
             # other batch sizes the table lists (not benchmarked)
             "resnet50 batch 32": lambda: zoo.resnet50_cfg(32, fuse_shortcut=True, in_place=True),
             "resnet50 batch 256": lambda: zoo.resnet50_cfg(256, fuse_shortcut=True, in_place=True),
             "vgg16 batch 64": lambda: zoo.vgg16_cfg(64), "alexnet batch 256": lambda: zoo.alexnet_cfg(256)}


@pytest.mark.parametrize("name", sorted(WORKLOADS))
def test_shipped_table_lists_every_convolution_of_the_benchmarked_networks(name):
    table = tune.read_table(TABLE)
    with Network(WORKLOADS[name](), device=-1) as net:          # dry run: shapes only
        convs = [i for i in range(net.num_layers) if net.layer_info(i)["kind"] == "convolutional_layer"]
        assert convs
        for i in convs:
            key = net.conv_problem(i)
            assert key in table, (name, i, key)
            if key[8]:
                assert table[key][0] != "strip"


def test_problem_key_of_fused_and_in_place_shortcuts():
    cfg = ("[net]\nbatch=3\nheight=8\nwidth=8\nchannels=4\nfuse_shortcut=1\nshortcut_in_place=1\n"
           "[convolutional]\nfilters=8\nsize=3\nstride=1\npadding=1\nactivation=relu\n"
           "[convolutional]\nfilters=6\nsize=3\nstride=1\npadding=1\nactivation=relu\n"
           "[convolutional]\nfilters=8\nsize=1\nstride=1\npadding=0\nactivation=linear\n"
           "[shortcut]\nhops=3\nactivation=relu\n"
           "[convolutional]\nfilters=16\nsize=3\nstride=2\npadding=1\nactivation=linear\n"
           "[shortcut]\nhops=2\nactivation=relu\n")
    with Network(cfg, device=-1) as net:
        assert net.conv_problem(0) == (4, 8, 8, 8, 3, 1, 1, 3, 0, 0, 0, 0)
        assert net.conv_problem(1) == (8, 8, 8, 6, 3, 1, 1, 3, 0, 0, 0, 0)
        assert net.conv_problem(2) == (6, 8, 8, 8, 1, 1, 0, 3, 8, 8, 8, 1)           # same shape: written over the connection
        assert net.conv_problem(4) == (8, 8, 8, 16, 3, 2, 1, 3, 8, 8, 8, 0)          # strided, wider: a tensor of its own
