"""Parity of exactly what bench.py times: ResNet-50 with shortcuts fused into the convolutions and the tile shape
and k-split found by the on-device search, at the benchmark's batch; the fused epilogue at the real stage-entry
shapes (strided and narrower residuals) through every tile shape; the gather modes the networks use
(tap-major, 1x1 vector) pinned bit for bit with one-hot filters; and the other configurations at their full
batch through properties that do not depend on size."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import bench  # noqa: E402  (synthetic weight generator and workload table shared with the benchmark)
from nebula_amd import zoo  # noqa: E402
from oracle import binding as ob  # noqa: E402

TOL = 1e-4


def rel(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(float(np.abs(b).max()), 1e-30))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32).ravel()


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


def bench_cfg(batch):
    """The cfg text bench.py's default workload builds."""
    cfg, b, _, _, _ = bench.workload("resnet50", batch)
    assert b == batch and "fuse_shortcut=1" in cfg and "shortcut_in_place=1" in cfg
    return cfg


def survives(net, i):
    """True when output(i) still holds layer i's own values after a pass (not a fused convolution, and not a tensor a
    later in-place shortcut wrote over)."""
    return net.output_writer(i) == i


def test_benched_resnet50_cfg_against_oracle_layer_by_layer():
    print("CASE benched resnet50 cfg (fused shortcuts) vs oracle at batch 2", flush=True)
    cfg = bench_cfg(2)
    rng = np.random.default_rng(2)
    net, blob = build(cfg)
    x = rng.standard_normal((2, 3, 224, 224)).astype(np.float32)
    want = oracle_forward(cfg, blob, x)
    net.set_input(x)
    net.forward()
    kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
    fused = overwritten = 0
    for i, k in enumerate(kinds):
        if k in ("cost_layer", "dropout_layer"):
            continue
        if k == "convolutional_layer" and kinds[i + 1] == "shortcut_layer":
            fused += 1          # no buffer of its own: its output IS the shortcut's, compared at the next index
            assert net.output_writer(i) >= i + 1
            continue
        if not survives(net, i):
            # a same-shape shortcut of the next block wrote its result over this one's tensor; what it holds now is
            # that later layer's output, which is compared at its own index
            overwritten += 1
            w = net.output_writer(i)
            assert kinds[i] == "shortcut_layer" and kinds[w] == "shortcut_layer" and w > i
            np.testing.assert_array_equal(bits(net.output(i)), bits(net.output(w)))
            continue
        r = rel(net.output(i), want[i].ravel())
        assert r <= TOL, (i, k, r)
    assert fused == 16
    assert overwritten == 12        # 16 blocks, 4 stages: the last block's output of every stage survives
    last = max(i for i, k in enumerate(kinds) if k == "connected_layer")
    np.testing.assert_array_equal(net.output(last).reshape(2, -1).argmax(1), want[last].reshape(2, -1).argmax(1))
    net.close()


def test_benched_resnet50_batch64_fused_searched_split():
    """bench.py's exact network at its exact batch: searched tile shapes and k-split, fused shortcuts.  Every image
    equals the same image through the same cfg at batch 2; every layer equals the unfused, unsplit network's."""
    print("CASE benched resnet50 b64: independence and fused-vs-unfused", flush=True)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((64, 3, 224, 224)).astype(np.float32)
    net64, blob = build(bench_cfg(64))
    net64.set_input(x)
    net64.forward()
    kinds = [net64.layer_info(i)["kind"] for i in range(net64.num_layers)]
    convs = [i for i, k in enumerate(kinds) if k == "convolutional_layer"]
    launches = [net64.conv_last_launch(i) for i in convs]
    assert all(v >= 0 for v, _ in launches)
    print("   k-split launches: %d of %d" % (sum(g > 1 for _, g in launches), len(launches)), flush=True)
    last = max(i for i, k in enumerate(kinds) if k == "connected_layer")
    logits64 = net64.output(last).reshape(64, 1000)
    probs64 = net64.output(last + 1).reshape(64, 1000)
    assert np.isfinite(logits64).all() and np.abs(probs64.sum(1) - 1).max() < 1e-4

    # (1) the unfused network with one summation order per layer (conv_split=0), layer by layer
    plain_cfg = zoo.resnet50_cfg(64).replace("[net]\n", "[net]\nconv_split=0\n", 1)
    plain, _ = build(plain_cfg)
    plain.set_input(x)
    plain.forward()
    worst = 0.0
    for i, k in enumerate(kinds):
        if k in ("cost_layer", "dropout_layer") or (k == "convolutional_layer" and kinds[i + 1] == "shortcut_layer"):
            continue
        if not survives(net64, i):
            continue
        r = rel(net64.output(i), plain.output(i))
        worst = max(worst, r)
        assert r <= TOL, (i, k, r)
    print("   worst layer rel diff fused+split vs unfused+unsplit: %.2e" % worst, flush=True)
    np.testing.assert_array_equal(logits64.argmax(1), plain.output(last).reshape(64, 1000).argmax(1))
    plain.close()

    # (2) per-image independence against the same cfg at batch 2 (which the oracle test above covers)
    net2, _ = build(bench_cfg(2))
    for lo in (0, 30, 62):
        net2.set_input(x[lo:lo + 2])
        net2.forward()
        logits2 = net2.output(last).reshape(2, 1000)
        assert rel(logits64[lo:lo + 2], logits2) <= TOL
        np.testing.assert_array_equal(logits64[lo:lo + 2].argmax(1), logits2.argmax(1))
    net2.close()

    # (3) pinning every layer to the launch the search chose reproduces the searched run bit for bit
    pinned, _ = build(bench_cfg(64))
    for i, (v, g) in zip(convs, launches):
        pinned.conv_pin_launch(i, v, g if g > 1 else 0)
    pinned.set_input(x)
    pinned.forward()
    assert [pinned.conv_last_launch(i) for i in convs] == launches
    np.testing.assert_array_equal(bits(pinned.output(last)), bits(net64.output(last)))
    pinned.close()

    # (4) the same launches with every shortcut writing into a buffer of its own: every element is read and written
    # by the same lane either way, so the surviving tensors agree bit for bit
    own_cfg = bench_cfg(64).replace("shortcut_in_place=1\n", "")
    own, _ = build(own_cfg)
    for i, (v, g) in zip(convs, launches):
        own.conv_pin_launch(i, v, g if g > 1 else 0)
    own.set_input(x)
    own.forward()
    assert all(own.output_writer(i) == i for i, k in enumerate(kinds) if k == "shortcut_layer")
    for i, k in enumerate(kinds):
        if k in ("shortcut_layer", "connected_layer", "avgpool_layer") and survives(net64, i):
            np.testing.assert_array_equal(bits(own.output(i)), bits(net64.output(i)), err_msg="layer %d" % i)
    own.close()
    net64.close()


# ResNet-50's last 1x1 of a block with the residual the network feeds it (B kept small for the oracle):
#   C, HW_in, F, conn_c, conn_hw
STAGE_RESIDUALS = [
    (64, 56, 256, 64, 56),        # block 1 of stage 2: residual = max-pool output, fewer channels
    (64, 56, 256, 256, 56),       # later blocks: same shape
    (128, 28, 512, 256, 56),      # entry of stage 3: strided (2x) and fewer channels
    (256, 14, 1024, 512, 28),     # entry of stage 4
    (512, 7, 2048, 1024, 14),     # entry of stage 5: odd plane (49 pixels)
    (512, 7, 2048, 2048, 7),      # stage 5, same shape, odd plane
]


@pytest.mark.parametrize("shape", STAGE_RESIDUALS)
@pytest.mark.parametrize("acts", [("linear", "relu"), ("leaky", "leaky")])
def test_fused_residual_at_stage_shapes_every_tile_shape(shape, acts):
    from nebula_amd import hip
    Cc, HW, F, cc, chw = shape
    act, post = acts
    B = 3
    print("CASE fused residual", shape, acts, flush=True)
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((B, Cc, HW, HW)).astype(np.float32)
    w = (rng.standard_normal((F, Cc, 1, 1)) * np.sqrt(2.0 / Cc)).astype(np.float32)
    bias = (rng.standard_normal(F) * 0.1).astype(np.float32)
    bnp = (rng.uniform(0.8, 1.2, F).astype(np.float32), (rng.standard_normal(F) * 0.1).astype(np.float32),
           rng.uniform(0.5, 1.5, F).astype(np.float32))
    conn = rng.standard_normal((B, cc, chw, chw)).astype(np.float32)
    assert ob.use_openblas(threads=16)
    try:
        want = ob.shortcut_forward(ob.conv_forward(x, w, bias, bnp, 1, 0, act), conn, post)
    finally:
        ob.use_custom_gemm()
        ob.set_threads(1)
    with hip.Ctx(0) as ctx:
        plan = ctx.conv_pack(w, bias, bnp, H=HW, W=HW, stride=1, pad=0, act=act)
        dx, dconn = ctx.array(x), ctx.array(conn)
        for v in range(hip.lib().nbl_conv2d_num_variants()):
            plan.set_variant(v)
            ref = None
            for split in (0, 1, 2, 5, 8):
                print("   variant", v, "split", split, flush=True)
                plan.set_split(split)
                got = plan.with_shortcut(dx, dconn, post).numpy()
                assert rel(got, want) <= TOL, (shape, v, split, rel(got, want))
                if split == 0:
                    ref = got
                else:
                    assert rel(got, ref) <= 1e-5, (shape, v, split)
        # the searched choice as the network would run it
        plan.set_variant(-1)
        plan.set_split(-1)
        assert rel(plan.with_shortcut(dx, dconn, post).numpy(), want) <= TOL


# One-hot filters: filter f holds a single 1.0 at (c_f, i_f, j_f), zero bias, linear activation.  Every product but
# one is an exact zero, so the kernel's output IS the patch element it gathered -- any summation order gives the
# same bits -- and must equal row (c_f*k + i_f)*k + j_f of the reference's im2col matrix (common/utils.cc:81-119).
ONE_HOT = [
    # C, H, W, k, stride, pad        gather mode the layer takes
    (32, 14, 14, 3, 1, 1),           # tap-major
    (16, 13, 11, 3, 2, 1),           # tap-major, strided, odd plane
    (48, 9, 9, 5, 1, 2),             # tap-major, 25 taps
    (16, 12, 12, 3, 1, 0),           # tap-major without padding
    (64, 8, 8, 1, 1, 0),             # 1x1 vector gather
    (96, 10, 6, 1, 1, 0),            # 1x1 vector gather, 3 k-tile pairs
    (3, 19, 19, 7, 2, 3),            # per-row table with bounds test (the stem's mode), and the strip kernel
    (3, 23, 23, 11, 4, 0),           # per-row table, no padding (AlexNet conv1's mode), and the strip kernel
    (3, 51, 38, 7, 2, 3),            # strip kernel: several tiles per image, the last one ragged
    (4, 30, 27, 3, 1, 1),            # strip kernel, 3x3 with padding (VGG's first layer has this form)
]


@pytest.mark.parametrize("geom", ONE_HOT)
def test_gather_bit_exact_through_the_convolution_kernel(geom):
    from nebula_amd import hip
    Cc, H, W, k, s, p = geom
    print("CASE one-hot filters", geom, flush=True)
    rng = np.random.default_rng(sum(geom))
    B, K = 3, Cc * k * k
    F = min(K, 200)
    rows = rng.permutation(K)[:F]
    rows[0], rows[1] = 0, K - 1              # first and last patch row always present
    w = np.zeros((F, K), np.float32)
    w[np.arange(F), rows] = 1.0
    w = w.reshape(F, Cc, k, k)
    x = rng.standard_normal((B, Cc, H, W)).astype(np.float32)
    cols = np.stack([ob.im2col(x[b], k, s, p) for b in range(B)])      # [B][K][OH*OW]
    want = cols[:, rows, :]
    with hip.Ctx(0) as ctx:
        plan = ctx.conv_pack(w, np.zeros(F, np.float32), None, H=H, W=W, stride=s, pad=p, act="linear")
        dx = ctx.array(x)
        nv = hip.lib().nbl_conv2d_num_variants()
        variants = list(range(nv))
        if hip.lib().nbl_conv2d_plan_set_variant(plan.p, nv) == 0:     # the strip kernel of layers with very few channels
            variants.append(nv)
        assert (nv in variants) == (Cc <= 4 and k > 1)
        for v in variants:
            plan.set_variant(v)
            for split in (0, 2, 8):
                plan.set_split(split)
                got = plan(dx).numpy().reshape(B, F, -1)
                # a padding tap read as 0.0 may come out as +0 or -0 only if a sign were invented: compare bits
                np.testing.assert_array_equal(bits(got), bits(want), err_msg="%r variant %d split %d" % (geom, v, split))


def _independence(name, batch, lo_list, xdist):
    """Images lo..lo+1 of the full batch against the same two images run alone."""
    cfg = zoo.WORKLOADS[name](batch)
    rng = np.random.default_rng(11)
    net, blob = build(cfg)
    c, h, w = net.input_shape
    x = (rng.random((batch, c, h, w)) if xdist == "uniform" else rng.standard_normal((batch, c, h, w))).astype(np.float32)
    net.set_input(x)
    net.forward()
    kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
    last = max(i for i, k in enumerate(kinds) if k == "connected_layer")
    logits = net.output(last).reshape(batch, -1)
    probs = net.output(last + 1).reshape(batch, -1)
    net.close()
    assert np.isfinite(logits).all() and np.abs(probs.sum(1) - 1).max() < 1e-4
    from nebula_amd.net import Network
    small = Network(zoo.WORKLOADS[name](2))
    small.load_weight_blob(blob)
    for lo in lo_list:
        small.set_input(x[lo:lo + 2])
        small.forward()
        l2 = small.output(last).reshape(2, -1)
        assert rel(logits[lo:lo + 2], l2) <= TOL, (name, lo, rel(logits[lo:lo + 2], l2))
        np.testing.assert_array_equal(logits[lo:lo + 2].argmax(1), l2.argmax(1))
    # the batch-2 network against the oracle closes the chain: full batch == batch 2 == reference algorithm
    want = oracle_forward(zoo.WORKLOADS[name](2), blob, x[:2])
    small.set_input(x[:2])
    small.forward()
    assert rel(small.output(last), want[last].ravel()) <= TOL
    small.close()


def test_alexnet_full_batch_128():
    print("CASE alexnet b128 independence", flush=True)
    _independence("alexnet", 128, (0, 63, 126), "uniform")


def test_vgg16_full_batch_32():
    print("CASE vgg16 b32 independence", flush=True)
    _independence("vgg16", 32, (0, 30), "normal")


def test_lstm_full_configuration_t64_b64_10000_way():
    """Config 5 at full size: T = 64, 64 sequences, 2 x LSTM 1024, 10000-way projection and softmax on the last
    step.  Sequences are independent of each other; two of them run alone (and against the oracle) must agree."""
    print("CASE lstm T=64 B=64 10000-way", flush=True)
    T, B = 64, 64
    cfg = zoo.lstm_cfg(batch=B, time_steps=T, last_step_only=True)
    rng = np.random.default_rng(13)
    net, blob = build(cfg, "lstm")
    x = rng.standard_normal((T, B, 1024)).astype(np.float32)
    net.set_input(x)
    net.forward()
    h2 = net.output(1).reshape(T, B, 1024)
    probs = net.output(3).reshape(T * B, -1)[:B]
    net.close()
    assert np.isfinite(h2).all() and np.abs(probs.sum(1) - 1).max() < 1e-4
    from nebula_amd.net import Network
    cfg2 = zoo.lstm_cfg(batch=2, time_steps=T, last_step_only=True)
    small = Network(cfg2)
    small.load_weight_blob(blob)
    want = oracle_forward(cfg2, blob, x[:, 62:64])
    for lo in (0, 62):
        xs = np.ascontiguousarray(x[:, lo:lo + 2])
        small.set_input(xs)
        small.forward()
        assert rel(h2[:, lo:lo + 2], small.output(1).reshape(T, 2, 1024)) <= TOL
        p2 = small.output(3).reshape(T * 2, -1)[:2]
        assert rel(probs[lo:lo + 2], p2) <= TOL
        np.testing.assert_array_equal(probs[lo:lo + 2].argmax(1), p2.argmax(1))
    assert rel(h2[:, 62:64], want[1].reshape(T, 2, 1024)) <= TOL
    assert rel(probs[62:64], want[3]) <= TOL
    np.testing.assert_array_equal(probs[62:64].argmax(1), want[3].argmax(1))
    small.close()


def test_last_step_only_reads_the_last_step_through_alias_layers():
    """[lstm] [dropout] [connected] with last_step_only: the connected layer must see the final time step although
    the layer between it and the LSTM only aliases the LSTM's buffer."""
    from nebula_amd.net import Network
    print("CASE last_step_only through dropout", flush=True)
    T, B, I, H, Cn = 5, 3, 12, 32, 9
    base = "[net]\nbatch=%d\ninput_size=%d\ntime_steps=%d\n%%s\n[lstm]\noutput=%d\nactivation=linear\n" % (B, I, T, H)
    tail = "\n[connected]\noutput=%d\nactivation=linear\n\n[softmax]\n" % Cn
    plain = base % "last_step_only=1" + tail
    dropped = base % "last_step_only=1" + "\n[dropout]\nprobability=0.5\n" + tail
    every = base % "" + "\n[dropout]\nprobability=0.5\n" + tail
    rng = np.random.default_rng(19)
    onet = ob.OracleNet(every)
    blob = np.concatenate([rng.uniform(-0.3, 0.3, shape).astype(np.float32).ravel()
                           for _, _, shape in ob.weight_layout(onet.specs)])
    onet.load_weights(blob)
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    ob.use_custom_gemm()
    want = onet.forward(x)[3].reshape(T, B, Cn)[T - 1]          # the oracle projects every step: take the last
    outs = {}
    for name, cfg, soft in (("plain", plain, 2), ("dropout", dropped, 3)):
        with Network(cfg) as net:
            net.load_weight_blob(blob)
            net.set_input(x)
            net.forward()
            outs[name] = net.output(soft).reshape(T * B, Cn)[:B]
        assert rel(outs[name], want) <= TOL, (name, rel(outs[name], want))
    np.testing.assert_array_equal(bits(outs["plain"]), bits(outs["dropout"]))


def test_fusion_is_skipped_when_a_later_shortcut_reads_the_convolution():
    """conv A, shortcut S1, conv B, shortcut S2 with hops reaching A: fusing A into S1 would leave S2 without A's own
    output.  The builder must keep that pair unfused; results equal the unfused network and the oracle."""
    from nebula_amd.net import Network
    print("CASE fusion guard", flush=True)
    conv = "\n[convolutional]\nfilters=8\nsize=3\nstride=1\npadding=1\nactivation=%s\n"
    body = (conv % "relu") + (conv % "linear") + "\n[shortcut]\nhops=2\nactivation=relu\n" + (conv % "linear") + \
        "\n[shortcut]\nhops=3\nactivation=leaky\n"          # second shortcut: 3 hops back = the second convolution
    head = "[net]\nbatch=2\nheight=10\nwidth=10\nchannels=4\n%s"
    cfg_plain, cfg_fused = head % "conv_split=0\n" + body, head % "conv_split=0\nfuse_shortcut=1\n" + body
    rng = np.random.default_rng(29)
    onet = ob.OracleNet(cfg_plain)
    blob = np.concatenate([(rng.standard_normal(shape) * 0.2).astype(np.float32).ravel()
                           for _, _, shape in ob.weight_layout(onet.specs)])
    onet.load_weights(blob)
    x = rng.standard_normal((2, 4, 10, 10)).astype(np.float32)
    ob.use_custom_gemm()
    want = onet.forward(x)
    outs = []
    for cfg in (cfg_plain, cfg_fused):
        with Network(cfg) as net:
            net.load_weight_blob(blob)
            net.set_input(x)
            net.forward()
            outs.append([net.output(i) for i in range(net.num_layers)])
    for i in range(5):
        assert rel(outs[0][i], want[i].ravel()) <= TOL, i
    # layer 1 (second convolution) is read by the last shortcut: it keeps its own output in the fused network too
    for i in (0, 1, 2, 4):
        np.testing.assert_array_equal(bits(outs[0][i]), bits(outs[1][i]), err_msg="layer %d" % i)


@pytest.mark.parametrize("shape", [(64, 56, 256), (256, 14, 1024), (512, 7, 2048), (96, 10, 80)])
def test_fused_residual_written_in_place(shape):
    """nbl_conv2d_shortcut_fwd with y == conn (same shape): the result replaces the residual and equals, bit for bit, what
    the same launch writes into a separate buffer -- for every tile shape, split and unsplit, and through the tile search
    (whose trial launches must not feed on their own output)."""
    from nebula_amd import hip
    Cc, HW, F = shape
    B = 4
    print("CASE in-place fused residual", shape, flush=True)
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((B, Cc, HW, HW)).astype(np.float32)
    w = (rng.standard_normal((F, Cc, 1, 1)) * np.sqrt(2.0 / Cc)).astype(np.float32)
    bias = (rng.standard_normal(F) * 0.1).astype(np.float32)
    conn = rng.standard_normal((B, F, HW, HW)).astype(np.float32)
    assert ob.use_openblas(threads=16)
    try:
        want = ob.shortcut_forward(ob.conv_forward(x, w, bias, None, 1, 0, "linear"), conn, "relu")
    finally:
        ob.use_custom_gemm()
        ob.set_threads(1)
    with hip.Ctx(0) as ctx:
        plan = ctx.conv_pack(w, bias, None, H=HW, W=HW, stride=1, pad=0, act="linear")
        dx = ctx.array(x)
        for v in list(range(hip.lib().nbl_conv2d_num_variants())) + [-1]:
            for split in ((0, 1, 5) if v >= 0 else (-1,)):
                print("   variant", v, "split", split, flush=True)
                plan.set_variant(v)
                plan.set_split(split)
                dconn, dy = ctx.array(conn), ctx.empty(conn.shape)
                if v < 0:
                    in_place = plan.with_shortcut(dx, dconn, "relu", out=dconn).numpy()       # the search runs here
                    launch = plan.last_launch()
                    dconn.upload(conn)
                    # (writing to a buffer of its own is another problem to the launch table: repeat the in-place launch)
                    plan.set_variant(launch[0])
                    plan.set_split(launch[1] if launch[1] > 1 else 0)
                    separate = plan.with_shortcut(dx, dconn, "relu", out=dy).numpy()
                    assert plan.last_launch() == launch
                else:
                    separate = plan.with_shortcut(dx, dconn, "relu", out=dy).numpy()
                    np.testing.assert_array_equal(bits(dconn.numpy()), bits(conn))              # residual untouched
                    in_place = plan.with_shortcut(dx, dconn, "relu", out=dconn).numpy()
                assert rel(separate, want) <= TOL, (shape, v, split)
                np.testing.assert_array_equal(bits(in_place), bits(separate), err_msg="%r variant %d split %d" % (shape, v, split))
                dconn.free(); dy.free()
        # a connection of another shape cannot be the output
        narrow = ctx.array(conn[:, : F // 2])
        rc = hip.lib().nbl_conv2d_shortcut_fwd(ctx.h, plan.p, dx.ptr, narrow.ptr, F // 2, HW, HW, narrow.ptr, B, hip.ACT["relu"])
        assert rc != 0 and b"alias" in hip.lib().nbl_last_error(ctx.h)
