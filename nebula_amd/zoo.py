"""network.cfg text for the networks the benchmarks are quoted on.

The topologies follow the reference's shipped cfgs (benchmarks/{alexnet,vgg,resnet,lstm}_large/network.cfg):
same layer sequence, filter counts, strides and paddings.  ResNet-50 is the reference's own variant:
bottlenecks [3,4,6,3] with the stride on the 3x3, `[shortcut] hops=4` residuals WITHOUT projection
convolutions, a 3x3/s2 maxpool with padding=0 and a 7x7/s7 average pool.
"""


def _net(batch, h, w, c, extra=""):
    return "[net]\nbatch=%d\nheight=%d\nwidth=%d\nchannels=%d\n%s" % (batch, h, w, c, extra)


def _conv(filters, size, stride, padding, activation, bn=False):
    return "\n[convolutional]\n%sfilters=%d\nsize=%d\nstride=%d\npadding=%d\nactivation=%s\n" % (
        "batch_normalize=1\n" if bn else "", filters, size, stride, padding, activation)


def _pool(kind, size, stride, padding=None):
    return "\n[%s]\nsize=%d\nstride=%d\n%s" % (kind, size, stride, "" if padding is None else "padding=%d\n" % padding)


def _fc(output, activation):
    return "\n[connected]\noutput=%d\nactivation=%s\n" % (output, activation)


_TAIL = "\n[softmax]\ngroups=1\n\n[cost]\ntype=l2\n"


def conv1_pool_cfg(batch=32, pool_index=False):
    """AlexNet conv1 + ReLU + 3x3/s2 maxpool.  pool_index: also keep the argmax table the reference's forward
    writes for its backward pass (a [net] key the reference ignores)."""
    return (_net(batch, 227, 227, 3, "pool_index=1\n" if pool_index else "") + _conv(96, 11, 4, 0, "relu")
            + _pool("maxpool", 3, 2, 0))


def alexnet_cfg(batch=128):
    s = _net(batch, 227, 227, 3)
    s += _conv(96, 11, 4, 0, "relu") + _pool("maxpool", 3, 2, 0)
    s += _conv(256, 5, 1, 2, "relu") + _pool("maxpool", 3, 2, 0)
    s += _conv(384, 3, 1, 1, "relu") + _conv(384, 3, 1, 1, "relu") + _conv(256, 3, 1, 1, "relu")
    s += _pool("maxpool", 3, 2, 0)
    s += _fc(4096, "relu") + "\n[dropout]\nprobability=0.5\n" + _fc(4096, "relu") + "\n[dropout]\nprobability=0.5\n"
    s += _fc(1000, "linear") + _TAIL
    return s


def vgg16_cfg(batch=32):
    s = _net(batch, 224, 224, 3)
    for filters, reps in ((64, 2), (128, 2), (256, 3), (512, 3), (512, 3)):
        for _ in range(reps):
            s += _conv(filters, 3, 1, 1, "relu")
        s += _pool("maxpool", 2, 2)
    s += _fc(4096, "relu") + "\n[dropout]\nprobability=0.5\n" + _fc(4096, "relu") + "\n[dropout]\nprobability=0.5\n"
    s += _fc(1000, "linear") + _TAIL
    return s


def resnet50_cfg(batch=64, activation="relu", fuse_shortcut=False, in_place=False):
    """fuse_shortcut: let each block's last convolution add the residual in its epilogue (a [net] key the
    reference ignores; results are bit-identical to the unfused network).  in_place: a fused shortcut whose
    connection has the output's shape writes its result over the connection's tensor (same values; the connection
    layer's own output is gone after the pass)."""
    s = _net(batch, 224, 224, 3, ("fuse_shortcut=1\n" if fuse_shortcut else "") + ("shortcut_in_place=1\n" if in_place else ""))
    s += _conv(64, 7, 2, 3, activation, bn=True) + _pool("maxpool", 3, 2, 0)
    for stage, (width, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3))):
        for block in range(blocks):
            stride = 2 if (stage > 0 and block == 0) else 1
            s += _conv(width, 1, 1, 0, activation, bn=True)
            s += _conv(width, 3, stride, 1, activation, bn=True)
            s += _conv(4 * width, 1, 1, 0, "linear", bn=True)
            s += "\n[shortcut]\nhops=4\nactivation=%s\n" % activation
    s += _pool("avgpool", 7, 7, 0) + _fc(1000, "linear") + _TAIL
    return s


def lstm_cfg(batch=64, time_steps=64, input_size=1024, hidden=1024, layers=2, classes=10000, last_step_only=False):
    """last_step_only: project and softmax the final time step only (a [net] key the reference ignores;
    the reference itself projects all T*B rows)."""
    s = "[net]\nbatch=%d\ninput_size=%d\ntime_steps=%d\n" % (batch, input_size, time_steps)
    if last_step_only:
        s += "last_step_only=1\n"
    for _ in range(layers):
        s += "\n[lstm]\noutput=%d\nactivation=linear\n" % hidden
    s += _fc(classes, "linear") + _TAIL
    return s


def rnn_cfg(batch=32, time_steps=40, input_size=8713, hidden=1024, layers=5, last_step_only=False):
    """benchmarks/rnn_large/network.cfg: five normalised [rnn] layers of 1024, projection back to the vocabulary."""
    s = "[net]\nbatch=%d\ninput_size=%d\ntime_steps=%d\n" % (batch, input_size, time_steps)
    if last_step_only:
        s += "last_step_only=1\n"
    for _ in range(layers):
        s += "\n[rnn]\nbatch_normalize=1\noutput=%d\nactivation=linear\n" % hidden
    s += _fc(input_size, "linear") + _TAIL
    return s


def dbn_cfg(batch=32):
    """benchmarks/dbn_large/network.cfg: four [rbm] layers (2000, 1000, 500, 30, logistic) on 3x128x128 inputs."""
    s = _net(batch, 128, 128, 3)
    for out in (2000, 1000, 500, 30):
        s += "\n[rbm]\noutput=%d\nk_step=1\nactivation=logistic\n" % out
    s += _fc(62, "linear") + _TAIL
    return s


def mlp_cfg(batch=32):
    """benchmarks/mlp_large/network.cfg: 2500-2000-1500-1000-500 relu, 62 classes, 3x128x128 inputs."""
    s = _net(batch, 128, 128, 3)
    for out in (2500, 2000, 1500, 1000, 500):
        s += _fc(out, "relu")
    s += _fc(62, "linear") + _TAIL
    return s


def synthetic_weights(layout, rng, dist, lstm_hidden=1024):
    """Synthetic weights in .wgh order from a network's own field table (Network.weight_layout()).  dist: 'he'
    (He-normal weights, N(0,0.01) bias, or for normalised layers beta N(0,0.1), gamma U[0.8,1.2], mean N(0,0.1),
    var U[0.5,1.5]) or 'lstm' (everything U[-1/sqrt(H), 1/sqrt(H)])."""
    import numpy as np
    normalised = {li for li, kind, _, _ in layout if kind == "scale"}
    parts = []
    for li, kind, count, fan_in in layout:
        if dist == "lstm":
            a = rng.uniform(-1, 1, count) / np.sqrt(lstm_hidden)
        elif kind == "weight":
            a = rng.standard_normal(count) * np.sqrt(2.0 / fan_in)
        elif kind == "bias":
            a = rng.standard_normal(count) * (0.1 if li in normalised else 0.01)
        elif kind == "scale":
            a = rng.uniform(0.8, 1.2, count)
        elif kind == "mean":
            a = rng.standard_normal(count) * 0.1
        else:
            a = rng.uniform(0.5, 1.5, count)
        parts.append(a.astype(np.float32))
    return np.concatenate(parts)


WORKLOADS = {
    "conv1": conv1_pool_cfg, "alexnet": alexnet_cfg, "vgg16": vgg16_cfg, "resnet50": resnet50_cfg, "lstm": lstm_cfg,
    "rnn": rnn_cfg, "dbn": dbn_cfg, "mlp": mlp_cfg,
}
