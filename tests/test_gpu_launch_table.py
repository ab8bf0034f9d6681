"""Convolution launches on the GPU come from the launch table: a benchmarked network launches the same way in every
process (bit-equal logits of two fresh processes, no pinning), a problem the table does not list is measured once and
then shared by every later plan, the search can be switched off, and batches beyond the kernels' 32-bit offsets run as
slices of whole images (the reference loops over images: models/layers/convolutional_layer.cc:374-399)."""
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import binding as ob  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ob.use_openblas(threads=8)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


def announce(*what):
    print("CASE", *what, flush=True)


@pytest.fixture()
def ctx():
    from nebula_amd import hip
    c = hip.Ctx(0)
    yield c
    c.close()
    hip.lib().nbl_launch_table_load(None)       # later tests see the shipped table again
    hip.lib().nbl_launch_table_set_search(1)


FRESH_PROCESS = """
import hashlib, sys
import numpy as np
sys.path.insert(0, %r)
from nebula_amd import zoo
from nebula_amd.net import Network
net = Network(zoo.resnet50_cfg(64, fuse_shortcut=True, in_place=True))
rng = np.random.default_rng(5)
net.load_weight_blob(zoo.synthetic_weights(net.weight_layout(), rng, "he"))
net.set_input(rng.standard_normal(net.batch_size * net.input_size).astype(np.float32))
net.forward()
net.sync()
convs = [i for i in range(net.num_layers) if net.layer_info(i)["kind"] == "convolutional_layer"]
logits = net.output(net.num_layers - 3)
assert np.isfinite(logits).all()
print("RESULT", hashlib.sha256(logits.tobytes()).hexdigest(), ",".join(sorted({net.conv_launch_source(i) for i in convs})),
      " ".join("%%d/%%d" %% net.conv_last_launch(i) for i in convs))
net.close()
"""


def test_two_fresh_processes_give_bit_equal_logits_without_pinning():
    announce("ResNet-50 b64, benchmarked cfg, two fresh processes")
    seen = []
    for run in range(2):
        out = subprocess.run([sys.executable, "-c", FRESH_PROCESS % ROOT], capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-2000:]
        line = [l for l in out.stdout.splitlines() if l.startswith("RESULT")][0].split(" ", 3)
        seen.append(line)
    assert seen[0][2] == "table", seen[0][2]          # every convolution launch came from the shipped file
    assert seen[0] == seen[1]


def test_unlisted_problem_is_measured_once_then_shared_and_can_be_saved(ctx, tmp_path):
    from nebula_amd import hip
    l = hip.lib()
    announce("unlisted problem: search, reuse, save, load")
    rng = np.random.default_rng(11)
    C_, H, F, B = 48, 30, 80, 24         # not a layer of any shipped network; big enough to be worth a search
    w = (rng.standard_normal((F, C_, 3, 3)) * 0.05).astype(np.float32)
    b = (rng.standard_normal(F) * 0.1).astype(np.float32)
    x = rng.standard_normal((B, C_, H, H)).astype(np.float32)
    want = ob.conv_forward(x, w, b, None, 1, 1, "relu")
    dx = ctx.array(x)
    before = l.nbl_launch_table_size()
    p1 = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="relu")
    y1 = p1(dx).numpy()
    assert p1.launch_source() == "searched" and l.nbl_launch_table_size() == before + 1
    assert rel(y1, want) <= 1e-4
    p2 = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="relu")        # an equal problem in a new plan: no second search
    y2 = p2(dx).numpy()
    assert p2.launch_source() == "searched" and l.nbl_launch_table_size() == before + 1
    assert p2.last_launch() == p1.last_launch()
    np.testing.assert_array_equal(bits(y2), bits(y1))
    # another batch is another problem
    p2(ctx.array(x[:7]))
    assert l.nbl_launch_table_size() == before + 2
    # the grown table written out and read back: the same launch, now an entry "from a file"
    path = str(tmp_path / "grown.txt")
    assert l.nbl_launch_table_save(path.encode()) == before + 2
    assert l.nbl_launch_table_load(path.encode()) == before + 2
    p3 = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="relu")
    y3 = p3(dx).numpy()
    assert p3.launch_source() == "table" and p3.last_launch() == p1.last_launch()
    np.testing.assert_array_equal(bits(y3), bits(y1))
    # a caller's pin wins over the table
    p3.set_variant(0)
    p3.set_split(0)
    p3(dx)
    assert p3.launch_source() == "pinned" and p3.last_launch() == (0, 1)


def test_search_switched_off_uses_the_cost_model_and_never_the_clock(ctx):
    from nebula_amd import hip
    l = hip.lib()
    announce("search off: cost model")
    l.nbl_launch_table_clear()
    l.nbl_launch_table_set_search(0)
    rng = np.random.default_rng(12)
    C_, H, F, B = 64, 28, 128, 16
    w = (rng.standard_normal((F, C_, 3, 3)) * 0.05).astype(np.float32)
    b = np.zeros(F, np.float32)
    x = rng.standard_normal((B, C_, H, H)).astype(np.float32)
    dx = ctx.array(x)
    outs, launches = [], []
    for _ in range(2):
        p = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="linear")
        outs.append(p(dx).numpy())
        assert p.launch_source() == "model"
        launches.append(p.last_launch())
    assert l.nbl_launch_table_size() == 0 and launches[0] == launches[1]
    np.testing.assert_array_equal(bits(outs[0]), bits(outs[1]))
    assert rel(outs[0], ob.conv_forward(x, w, b, None, 1, 1, "linear")) <= 1e-4


def replicate(ctx, block, times):
    """A device tensor holding `times` copies of the host array `block` back to back (filled on the device)."""
    from nebula_amd import hip
    out = ctx.empty((times * block.shape[0],) + block.shape[1:])
    src = ctx.array(block)
    for t in range(times):
        ctx.check(hip.lib().nbl_copy_d2d(ctx.h, out.ptr + t * src.nbytes, src.ptr, src.nbytes))
    src.free()
    return out


def rows(ctx, arr, first, count):
    """Images first .. first + count - 1 of a device tensor, on the host."""
    from nebula_amd import hip
    per = int(np.prod(arr.shape[1:]))
    out = np.empty((count,) + arr.shape[1:], np.float32)
    ctx.check(hip.lib().nbl_d2h(ctx.h, out.ctypes.data, arr.ptr + first * per * 4, out.nbytes))
    return out


def test_batch_beyond_32_bit_offsets_runs_as_slices_of_images(ctx):
    """VGG-16's second convolution (64 -> 64, 3x3 on 224x224) at batch 192: 616 M input elements, more than one launch can
    address.  With the tile shape pinned and no k-split every output element is the same sum in the same order whatever
    the batch, so image i of the big batch must equal that image convolved alone, bit for bit."""
    announce("conv 64x224x224 -> 64, batch 192 (two launches)")
    rng = np.random.default_rng(13)
    C_, H, F, B, distinct = 64, 224, 64, 192, 4
    w = (rng.standard_normal((F, C_, 3, 3)) * np.sqrt(2.0 / (9 * C_))).astype(np.float32)
    b = (rng.standard_normal(F) * 0.01).astype(np.float32)
    block = rng.standard_normal((distinct, C_, H, H)).astype(np.float32)
    x = replicate(ctx, block, B // distinct)
    assert x.size >= 1 << 29
    y = ctx.empty((B, F, H, H))
    plan = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=1, act="relu")
    plan.set_variant(0)
    plan.set_split(0)
    plan(x, out=y)
    alone = plan(ctx.array(block)).numpy()
    for first in (0, 92, 96, B - distinct):           # images on both sides of the cut between the two launches
        got = rows(ctx, y, first, distinct)
        np.testing.assert_array_equal(bits(got), bits(alone))
    assert rel(alone[:1], ob.conv_forward(block[:1], w, b, None, 1, 1, "relu")) <= 1e-4
    # the default path (table or search per slice) agrees to rounding
    plan.set_variant(-1)
    plan.set_split(-1)
    y.zero()
    plan(x, out=y)
    assert rel(rows(ctx, y, B - distinct, distinct), alone) <= 1e-5


@pytest.mark.parametrize("in_place", [False, True])
def test_fused_residual_beyond_32_bit_offsets(ctx, in_place):
    """A 1x1 layer with a same-shape residual whose tensors pass 2^29 input elements: the residual (and, in place, the
    output) must be cut at the same images as the input."""
    announce("conv 1x1 8 -> 8 on 512x512 + residual, batch 300, in place" if in_place else "conv 1x1 8 -> 8 on 512x512 + residual, batch 300")
    rng = np.random.default_rng(14)
    C_, H, F, B, distinct = 8, 512, 8, 300, 4
    w = (rng.standard_normal((F, C_, 1, 1)) * 0.3).astype(np.float32)
    b = (rng.standard_normal(F) * 0.1).astype(np.float32)
    block = rng.standard_normal((distinct, C_, H, H)).astype(np.float32)
    rblock = rng.standard_normal((distinct, F, H, H)).astype(np.float32)
    x = replicate(ctx, block, B // distinct)
    conn = replicate(ctx, rblock, B // distinct)
    assert x.size >= 1 << 29
    plan = ctx.conv_pack(w, b, None, H=H, W=H, stride=1, pad=0, act="linear")
    plan.set_variant(4)
    plan.set_split(0)
    y = conn if in_place else ctx.empty((B, F, H, H))
    plan.with_shortcut(x, conn, "relu", out=y)
    want = ob.shortcut_forward(ob.conv_forward(block, w, b, None, 1, 0, "linear"), rblock, "relu")
    for first in (0, 148, 152, B - distinct):
        got = rows(ctx, y, first, distinct)
        assert rel(got, want) <= 1e-4
        np.testing.assert_array_equal(bits(got), bits(rows(ctx, y, 0, distinct)))
