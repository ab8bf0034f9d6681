"""TEST INFRASTRUCTURE ONLY: ctypes bindings for the CPU oracle (oracle/libnebula_oracle.so)
and, where it exists, for the compiled unmodified reference (oracle/_ref/libnebula_ref.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module; the
product package never does.

Besides the per-function bindings it holds `OracleNet`, which walks a Nebula network.cfg the
way models/networks/network.cc:57-63 walks its layer list and calls the oracle per layer, and
`RefNet`, the same view over the reference build.
"""
import ctypes as C
import glob
import os
import subprocess
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libnebula_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libnebula_ref.so")
REFERENCE_ROOT = "/root/reference"

# activation_type_t, common/def.h:62-96
ACT_NAMES = ["undefined_activation", "elu", "hardtan", "leaky", "lhtan", "linear", "loggy", "logistic",
             "plse", "ramp", "relie", "relu", "stair", "tanh"]
ACT = {n: i for i, n in enumerate(ACT_NAMES)}

_f32p = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint)
_u = C.c_uint


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def build_oracle(force=False):
    """Compile the C restatement (gcc, ~1 s)."""
    if force or not os.path.exists(ORACLE_SO) or \
            os.path.getmtime(ORACLE_SO) < os.path.getmtime(os.path.join(HERE, "nebula_oracle.c")):
        subprocess.check_call(["make", "-C", HERE, "oracle"], stdout=subprocess.DEVNULL)
    return ORACLE_SO


def build_ref(force=False):
    """Compile the unmodified reference + harness; only where the reference tree exists."""
    if not os.path.isdir(REFERENCE_ROOT):
        return None
    if force or not os.path.exists(REF_SO):
        subprocess.check_call(["make", "-C", HERE, "ref"], stdout=subprocess.DEVNULL)
    return REF_SO


_oracle = None


def oracle():
    global _oracle
    if _oracle is None:
        build_oracle()
        lib = C.CDLL(ORACLE_SO)
        lib.orc_set_threads.argtypes = [_u]
        lib.orc_get_threads.restype = _u
        lib.orc_use_openblas.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p]
        lib.orc_use_openblas.restype = C.c_int
        lib.orc_im2col.argtypes = [_f32p, _u, _u, _u, _u, _u, _u, _f32p]
        lib.orc_gemm.argtypes = [C.c_int, C.c_int, _u, _u, _u, C.c_float, _f32p, _u, _f32p, _u,
                                 C.c_float, _f32p, _u]
        lib.orc_forward_bias.argtypes = [_f32p, _f32p, _u, _u, _u]
        lib.orc_batchnorm_normalize.argtypes = [_f32p, _f32p, _f32p, _u, _u, _u]
        lib.orc_batchnorm_scale_down.argtypes = [_f32p, _f32p, _u, _u, _u]
        lib.orc_activate.argtypes = [_u, _f32p, _u]
        lib.orc_activate.restype = C.c_int
        for f in ("orc_conv_out_dim",):
            getattr(lib, f).argtypes = [_u, _u, _u, _u]
            getattr(lib, f).restype = _u
        lib.orc_pool_out_dim.argtypes = [_u, _u, _u]
        lib.orc_pool_out_dim.restype = _u
        lib.orc_pool_default_padding.argtypes = [_u]
        lib.orc_pool_default_padding.restype = _u
        lib.orc_conv_forward.argtypes = [_f32p] * 8 + [_u] * 9
        lib.orc_connected_forward.argtypes = [_f32p] * 7 + [_u] * 4
        lib.orc_maxpool_forward.argtypes = [_f32p, _f32p, _u32p] + [_u] * 7
        lib.orc_avgpool_forward.argtypes = [_f32p, _f32p] + [_u] * 7
        lib.orc_shortcut_forward.argtypes = [_f32p, _f32p, _f32p] + [_u] * 8
        lib.orc_softmax_forward.argtypes = [_f32p, _f32p, _u, _u]
        lib.orc_target_prob_sum.argtypes = [_f32p, C.c_void_p, _u, _u]
        lib.orc_target_prob_sum.restype = C.c_float
        lib.orc_perplexity.argtypes = [C.c_float, _u]
        lib.orc_perplexity.restype = C.c_float
        lib.orc_image_to_input.argtypes = [C.c_void_p, _u, _u, _u, _f32p, _u, _u]
        lib.orc_resize_linear_u8.argtypes = [C.c_void_p, _u, _u, _u, C.c_void_p, _u, _u]
        lib.orc_linear_taps.argtypes = [_u, _u, C.c_int, C.c_void_p, C.c_void_p]
        pp = C.POINTER(_f32p)
        lib.orc_rnn_forward.argtypes = [_f32p, pp, pp, pp, pp, pp, _f32p, _u, _u, _u, _u, _u]
        lib.orc_topk_matches.argtypes = [_f32p, C.c_void_p, _u, _u, _u]
        lib.orc_topk_matches.restype = _u
        lib.orc_lstm_forward.argtypes = [_f32p, pp, pp, pp, pp, pp, _f32p, _f32p, _u, _u, _u, _u, _u]
        _oracle = lib
    return _oracle


def find_openblas():
    """The LP64 OpenBLAS that ships inside scipy (exports scipy_cblas_sgemm), or None."""
    try:
        import scipy
    except ImportError:
        return None
    root = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs")
    hits = sorted(glob.glob(os.path.join(root, "libscipy_openblas-*.so")))
    return hits[0] if hits else None


def use_openblas(threads=None):
    """Switch the oracle's GEMM to OpenBLAS (the reference's default BLAS). Returns True on success."""
    so = find_openblas()
    if so is None:
        return False
    rc = oracle().orc_use_openblas(so.encode(), b"scipy_cblas_sgemm", b"scipy_openblas_set_num_threads")
    if rc == 0 and threads:
        set_threads(threads)
    return rc == 0


def use_custom_gemm():
    oracle().orc_use_custom_gemm()


def set_threads(n):
    oracle().orc_set_threads(int(n))


# ------------------------------------------------------------------------------------------------
# numpy-level wrappers
# ------------------------------------------------------------------------------------------------
def conv_out_dim(n, k, s, p):
    return oracle().orc_conv_out_dim(n, k, s, p)


def pool_out_dim(n, s, p):
    return oracle().orc_pool_out_dim(n, s, p)


def im2col(im, k, s, p):
    im = _f32(im)
    c, h, w = im.shape
    oh, ow = conv_out_dim(h, k, s, p), conv_out_dim(w, k, s, p)
    col = np.empty((c * k * k, oh * ow), np.float32)
    oracle().orc_im2col(_fp(im), c, h, w, k, s, p, _fp(col))
    return col


def gemm(ta, tb, A, B, Cmat, alpha=1.0, beta=1.0):
    A, B = _f32(A), _f32(B)
    out = _f32(Cmat).copy()
    M, N = out.shape
    K = A.shape[0] if ta else A.shape[1]
    oracle().orc_gemm(int(ta), int(tb), M, N, K, alpha, _fp(A), A.shape[1], _fp(B), B.shape[1], beta,
                      _fp(out), N)
    return out


def activate(act, x):
    out = _f32(x).copy()
    rc = oracle().orc_activate(ACT[act] if isinstance(act, str) else act, _fp(out), out.size)
    if rc != 0:
        raise ValueError("undefined activation type")
    return out


def conv_forward(x, w, bias, bn=None, stride=1, padding=0, act="linear"):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    B, Cc, H, W = x.shape
    F, _, k, _ = w.shape
    oh, ow = conv_out_dim(H, k, stride, padding), conv_out_dim(W, k, stride, padding)
    y = np.empty((B, F, oh, ow), np.float32)
    ws = np.empty(Cc * k * k * oh * ow, np.float32)
    sc, mu, var = (None, None, None) if bn is None else [_f32(a) for a in bn]
    oracle().orc_conv_forward(_fp(x), _fp(w), _fp(bias), _fp(sc), _fp(mu), _fp(var), _fp(y), _fp(ws),
                              B, Cc, H, W, F, k, stride, padding, ACT[act])
    return y


def connected_forward(x, w, bias, bn=None, act="linear"):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    B = x.shape[0]
    x2 = x.reshape(B, -1)
    O, I = w.shape
    assert x2.shape[1] == I
    y = np.empty((B, O), np.float32)
    sc, mu, var = (None, None, None) if bn is None else [_f32(a) for a in bn]
    oracle().orc_connected_forward(_fp(x2), _fp(w), _fp(bias), _fp(sc), _fp(mu), _fp(var), _fp(y),
                                   B, I, O, ACT[act])
    return y


def maxpool_forward(x, k, s, p):
    x = _f32(x)
    B, Cc, H, W = x.shape
    oh, ow = pool_out_dim(H, s, p), pool_out_dim(W, s, p)
    y = np.empty((B, Cc, oh, ow), np.float32)
    idx = np.empty((B, Cc, oh, ow), np.uint32)
    oracle().orc_maxpool_forward(_fp(x), _fp(y), idx.ctypes.data_as(_u32p), B, Cc, H, W, k, s, p)
    return y, idx


def avgpool_forward(x, k, s, p):
    x = _f32(x)
    B, Cc, H, W = x.shape
    oh, ow = pool_out_dim(H, s, p), pool_out_dim(W, s, p)
    y = np.empty((B, Cc, oh, ow), np.float32)
    oracle().orc_avgpool_forward(_fp(x), _fp(y), B, Cc, H, W, k, s, p)
    return y


def shortcut_forward(prev, conn, act="linear"):
    prev, conn = _f32(prev), _f32(conn)
    B, oc, oh, ow = prev.shape
    _, ic, ih, iw = conn.shape
    out = np.empty_like(prev)
    oracle().orc_shortcut_forward(_fp(prev), _fp(conn), _fp(out), B, ic, ih, iw, oc, oh, ow, ACT[act])
    return out


def target_prob_sum(probs, targets):
    probs = _f32(probs); targets = np.ascontiguousarray(targets, np.uint32)
    rows, n = probs.shape
    return float(oracle().orc_target_prob_sum(_fp(probs), targets.ctypes.data, rows, n))


def perplexity(cumulative_cost, rows_seen):
    return float(oracle().orc_perplexity(cumulative_cost, rows_seen))


def image_to_input(img, dst_h, dst_w):
    """img: uint8 [h][w][c] -> float32 [c][dst_h][dst_w] (convolutional_t::load_data contract)."""
    img = np.ascontiguousarray(img, np.uint8)
    h, w, c = img.shape
    out = np.empty((c, dst_h, dst_w), np.float32)
    oracle().orc_image_to_input(img.ctypes.data, h, w, c, _fp(out), dst_h, dst_w)
    return out


def linear_taps(dst_n, src_n, clamp_weight):
    """First source index and the two 11-bit weights of every destination pixel along one axis."""
    ofs = np.empty(dst_n, np.int32)
    w = np.empty((dst_n, 2), np.int16)
    oracle().orc_linear_taps(dst_n, src_n, int(clamp_weight), ofs.ctypes.data, w.ctypes.data)
    return ofs, w


def resize_linear_u8(img, dst_h, dst_w):
    img = np.ascontiguousarray(img, np.uint8)
    h, w, c = img.shape
    out = np.empty((dst_h, dst_w, c), np.uint8)
    oracle().orc_resize_linear_u8(img.ctypes.data, h, w, c, out.ctypes.data, dst_h, dst_w)
    return out


def softmax_forward(x):
    x = _f32(x)
    rows = x.shape[0]
    x2 = x.reshape(rows, -1)
    y = np.empty_like(x2)
    oracle().orc_softmax_forward(_fp(x2), _fp(y), rows, x2.shape[1])
    return y


def _ptr_array(arrs):
    if arrs is None:
        return None
    return (_f32p * len(arrs))(*[_fp(a) for a in arrs])


def lstm_forward(x, weight, bias, bn=None, act="linear", want_cell=False):
    """x [T,B,I]; weight/bias: 8 arrays in file order iW,fW,oW,cW,iU,fU,oU,cU; bn = (scale8, mean8, var8)."""
    x = _f32(x)
    T, B, I = x.shape
    weight = [_f32(w) for w in weight]
    bias = [_f32(b) for b in bias]
    H = weight[0].shape[0]
    y = np.empty((T, B, H), np.float32)
    cell = np.empty((T, B, H), np.float32) if want_cell else None
    if bn is not None:
        bn = [[_f32(a) for a in grp] for grp in bn]
    sc, mu, var = (None, None, None) if bn is None else bn
    oracle().orc_lstm_forward(_fp(x), _ptr_array(weight), _ptr_array(bias), _ptr_array(sc), _ptr_array(mu),
                              _ptr_array(var), _fp(y), _fp(cell), T, B, I, H, ACT[act])
    return (y, cell) if want_cell else y


def rnn_forward(x, weight, bias, bn=None, act="linear"):
    """x [T,B,I]; weight/bias: 3 arrays in file order input, hidden, output gate; bn = (scale3, mean3, var3)."""
    x = _f32(x)
    T, B, I = x.shape
    weight = [_f32(w) for w in weight]
    bias = [_f32(b) for b in bias]
    O = weight[0].shape[0]
    y = np.empty((T, B, O), np.float32)
    if bn is not None:
        bn = [[_f32(a) for a in grp] for grp in bn]
    sc, mu, var = (None, None, None) if bn is None else bn
    oracle().orc_rnn_forward(_fp(x), _ptr_array(weight), _ptr_array(bias), _ptr_array(sc), _ptr_array(mu),
                             _ptr_array(var), _fp(y), T, B, I, O, ACT[act])
    return y


def topk_matches(probs, labels, k):
    probs = _f32(probs); labels = np.ascontiguousarray(labels, np.uint32)
    rows, n = probs.shape
    return int(oracle().orc_topk_matches(_fp(probs), labels.ctypes.data, rows, n, k))


# ------------------------------------------------------------------------------------------------
# network.cfg handling (common/config.cc:44-75: spaces stripped, '#' comments, keys AND values
# lower-cased, unknown keys ignored)
# ------------------------------------------------------------------------------------------------
def parse_cfg(text):
    sections = []
    for line in text.splitlines():
        line = line.replace(" ", "")
        if not line or line[0] == "#":
            continue
        if line[0] == "[":
            sections.append((line[1:-1], {}))
        else:
            eq = line.find("=")
            if eq < 0:
                raise ValueError("invalid config: " + line)
            key, val = line[:eq].lower(), line[eq + 1:].lower()
            sections[-1][1].setdefault(key, val)   # std::map::insert keeps the first value
    return sections


def _stream_uint(val, default):
    """`stringstream >> unsigned`: leading digits or keep the default."""
    digits = ""
    for ch in val:
        if ch.isdigit():
            digits += ch
        else:
            break
    return int(digits) if digits else default


class LayerSpec:
    def __init__(self, kind, **kw):
        self.kind = kind
        self.__dict__.update(kw)

    def __repr__(self):
        return "LayerSpec(%s)" % ", ".join("%s=%r" % kv for kv in self.__dict__.items())


def plan_network(cfg_text, batch=None):
    """cfg -> (net dict, [LayerSpec]) with every shape resolved by the reference's rules
    (convolutional.cc:52-122 / recurrent.cc:115-175 and each layer's init())."""
    sections = parse_cfg(cfg_text)
    net = {"batch": 1, "time_steps": 1, "height": 1, "width": 1, "channels": 1, "recurrent": False}
    specs = []
    cur = None   # (c, h, w, size) of the running output
    for name, kv in sections:
        g = lambda k, d: _stream_uint(kv[k], d) if k in kv else d
        if name == "net":
            net["batch"] = g("batch", 1) if batch is None else batch
            net["height"], net["width"], net["channels"] = g("height", 1), g("width", 1), g("channels", 1)
            net["input_size"] = net["height"] * net["width"] * net["channels"]
            if "time_steps" in kv:
                net["recurrent"] = True
                net["time_steps"] = g("time_steps", 1)
                # harness extension (a key the reference ignores): layers after the last LSTM see the final step only
                net["last_step_only"] = bool(g("last_step_only", 0))
                net["input_size"] = g("input_size", 0)
                cur = (1, 1, 1, net["input_size"])
            else:
                cur = (net["channels"], net["height"], net["width"], net["input_size"])
            net["num_threads"] = g("num_threads", 1)
            continue
        c, h, w, size = cur
        act = kv.get("activation")
        if act is not None and act not in ACT:
            raise ValueError("unknown activation " + act)
        bn = bool(g("batch_normalize", 0))
        if name == "convolutional":
            F, k, s, p = g("filters", 1), g("size", 1), g("stride", 1), g("padding", 0)
            oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
            specs.append(LayerSpec(name, C=c, H=h, W=w, F=F, k=k, s=s, p=p, bn=bn, act=act, out=(F, oh, ow)))
            cur = (F, oh, ow, F * oh * ow)
        elif name == "connected":
            O = g("output", 0)
            specs.append(LayerSpec(name, I=size, O=O, bn=bn, act=act, out=(1, 1, 1)))
            cur = (1, 1, 1, O)
        elif name in ("maxpool", "avgpool"):
            s = g("stride", 1)
            k = g("size", s)
            p = g("padding", (k - 1) // 2)
            oh, ow = (h + 2 * p) // s, (w + 2 * p) // s
            specs.append(LayerSpec(name, C=c, H=h, W=w, k=k, s=s, p=p, out=(c, oh, ow)))
            cur = (c, oh, ow, c * oh * ow)
        elif name == "shortcut":
            hops = g("hops", 0)
            src = len(specs) - hops    # index of the layer `hops` back from this one
            if src < 0:
                raise ValueError("shortcut hops reach before the first layer")
            specs.append(LayerSpec(name, hops=hops, src=src, act=act, out=(c, h, w)))
        elif name == "softmax":
            specs.append(LayerSpec(name, n=size, out=(c, h, w)))
        elif name == "dropout":
            specs.append(LayerSpec(name, out=(1, 1, 1)))   # identity at inference, dropout_layer.cc:72
            cur = (1, 1, 1, size)
        elif name == "cost":
            specs.append(LayerSpec(name, out=(c, h, w)))
        elif name == "lstm":
            O = g("output", 0)
            specs.append(LayerSpec(name, I=size, H=O, bn=bn, act=act, out=(1, 1, 1)))
            cur = (1, 1, 1, O)
        elif name == "rnn":
            O = g("output", 0)
            specs.append(LayerSpec(name, I=size, O=O, bn=bn, act=act, out=(1, 1, 1)))
            cur = (1, 1, 1, O)
        elif name == "rbm":     # rbm_layer.cc:70-90, forward = connected without batchnorm (:345-374)
            O = g("output", 0)
            specs.append(LayerSpec(name, I=size, O=O, bn=False, act=act, out=(1, 1, 1)))
            cur = (1, 1, 1, O)
        else:
            raise ValueError("unknown layer type " + name)
        specs[-1].out_size = cur[3] if name not in ("shortcut", "softmax", "cost") else size
        specs[-1].shape = cur[:3]
    return net, specs


def weight_layout(specs):
    """[(layer index, field name, shape)] in .wgh byte order (network.cc:108-110 and each init_weight)."""
    fields = []
    for li, sp in enumerate(specs):
        if sp.kind == "convolutional":
            fields += [(li, "bias", (sp.F,)), (li, "weight", (sp.F, sp.C, sp.k, sp.k))]
            if sp.bn:
                fields += [(li, "scale", (sp.F,)), (li, "mean", (sp.F,)), (li, "var", (sp.F,))]
        elif sp.kind == "connected":
            fields += [(li, "bias", (sp.O,)), (li, "weight", (sp.O, sp.I))]
            if sp.bn:
                fields += [(li, "scale", (sp.O,)), (li, "mean", (sp.O,)), (li, "var", (sp.O,))]
        elif sp.kind == "rbm":          # rbm_layer.cc:150-153: hidden_bias, weight
            fields += [(li, "bias", (sp.O,)), (li, "weight", (sp.O, sp.I))]
        elif sp.kind == "rnn":          # rnn_layer.cc:73-77: input, hidden, output gate, each a connected layer's fields
            for sub, fan_in in (("in", sp.I), ("hid", sp.O), ("out", sp.O)):
                fields += [(li, sub + ".bias", (sp.O,)), (li, sub + ".weight", (sp.O, fan_in))]
                if sp.bn:
                    fields += [(li, sub + ".scale", (sp.O,)), (li, sub + ".mean", (sp.O,)), (li, sub + ".var", (sp.O,))]
        elif sp.kind == "lstm":
            for sub in ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU"):
                fan_in = sp.H if sub[1] == "W" else sp.I
                fields += [(li, sub + ".bias", (sp.H,)), (li, sub + ".weight", (sp.H, fan_in))]
                if sp.bn:
                    fields += [(li, sub + ".scale", (sp.H,)), (li, sub + ".mean", (sp.H,)),
                               (li, sub + ".var", (sp.H,))]
    return fields


def split_weights(specs, blob):
    """flat fp32 .wgh contents -> {layer index: {field: array}}"""
    blob = np.asarray(blob, np.float32).ravel()
    out, pos = {}, 0
    for li, name, shape in weight_layout(specs):
        n = int(np.prod(shape))
        out.setdefault(li, {})[name] = blob[pos:pos + n].reshape(shape)
        pos += n
    if pos != blob.size:
        raise ValueError("weight blob has %d floats, layout needs %d" % (blob.size, pos))
    return out


class OracleNet:
    """Forward of a whole cfg-described network through the C oracle, layer by layer."""

    def __init__(self, cfg_text, batch=None):
        self.net, self.specs = plan_network(cfg_text, batch)
        self.weights = {}

    def load_weights(self, blob):
        self.weights = split_weights(self.specs, blob)

    def forward(self, x):
        """x: [B,C,H,W] (or [T,B,I] for recurrent nets).  Returns the list of layer outputs."""
        outs = []
        cur = _f32(x)
        T = self.net["time_steps"]
        for li, sp in enumerate(self.specs):
            wt = self.weights.get(li, {})
            if sp.kind == "convolutional":
                bn = (wt["scale"], wt["mean"], wt["var"]) if sp.bn else None
                cur = conv_forward(cur, wt["weight"], wt["bias"], bn, sp.s, sp.p, sp.act)
            elif sp.kind == "connected":
                bn = (wt["scale"], wt["mean"], wt["var"]) if sp.bn else None
                rows = cur.shape[0] * (cur.shape[1] if self.net["recurrent"] and cur.ndim == 3 else 1)
                cur = connected_forward(cur.reshape(rows, -1), wt["weight"], wt["bias"], bn, sp.act)
            elif sp.kind == "maxpool":
                cur, idx = maxpool_forward(cur, sp.k, sp.s, sp.p)
                sp.last_index = idx
            elif sp.kind == "avgpool":
                cur = avgpool_forward(cur, sp.k, sp.s, sp.p)
            elif sp.kind == "shortcut":
                cur = shortcut_forward(cur, outs[sp.src], sp.act)
            elif sp.kind == "softmax":
                cur = softmax_forward(cur.reshape(-1, sp.n))
            elif sp.kind in ("dropout", "cost"):
                pass
            elif sp.kind == "rbm":
                rows = cur.shape[0] * (cur.shape[1] if self.net["recurrent"] and cur.ndim == 3 else 1)
                cur = connected_forward(cur.reshape(rows, -1), wt["weight"], wt["bias"], None, sp.act)
            elif sp.kind == "rnn":
                subs = ("in", "hid", "out")
                bn = None
                if sp.bn:
                    bn = ([wt[q + ".scale"] for q in subs], [wt[q + ".mean"] for q in subs], [wt[q + ".var"] for q in subs])
                cur = rnn_forward(cur.reshape(T, -1, sp.I), [wt[q + ".weight"] for q in subs],
                                  [wt[q + ".bias"] for q in subs], bn, sp.act)
            elif sp.kind == "lstm":
                subs = ("iW", "fW", "oW", "cW", "iU", "fU", "oU", "cU")
                bn = None
                if sp.bn:
                    bn = ([wt[s + ".scale"] for s in subs], [wt[s + ".mean"] for s in subs],
                          [wt[s + ".var"] for s in subs])
                cur = lstm_forward(cur.reshape(T, -1, sp.I), [wt[s + ".weight"] for s in subs],
                                   [wt[s + ".bias"] for s in subs], bn, sp.act)
                last_lstm = max(i for i, q in enumerate(self.specs) if q.kind == "lstm")
                if self.net.get("last_step_only") and li == last_lstm:
                    outs.append(cur)
                    cur = cur[-1:]          # [1, B, H]: only the final step feeds the rest
                    continue
            outs.append(cur)
        return outs


# ------------------------------------------------------------------------------------------------
# The compiled reference (authoring container only)
# ------------------------------------------------------------------------------------------------
_ref = None


def ref():
    """ctypes handle of oracle/_ref/libnebula_ref.so, or None where it cannot exist."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO) and build_ref() is None:
            return None
        lib = C.CDLL(REF_SO)
        lib.ref_net_create.argtypes = [C.c_char_p]
        lib.ref_net_create.restype = C.c_void_p
        lib.ref_net_num_layers.argtypes = [C.c_void_p]
        lib.ref_net_num_layers.restype = _u
        lib.ref_net_dims.argtypes = [C.c_void_p, _u32p]
        lib.ref_net_layer_dims.argtypes = [C.c_void_p, _u, _u32p]
        lib.ref_net_load_weights.argtypes = [C.c_void_p, C.c_char_p]
        lib.ref_net_forward.argtypes = [C.c_void_p, _f32p]
        lib.ref_net_output.argtypes = [C.c_void_p, _u]
        lib.ref_net_output.restype = _f32p
        lib.ref_net_pool_index.argtypes = [C.c_void_p, _u]
        lib.ref_net_pool_index.restype = _u32p
        lib.ref_im2col.argtypes = [_f32p, _u, _u, _u, _u, _u, _u, _f32p, _u]
        lib.ref_gemm.argtypes = [C.c_int, C.c_int, _u, _u, _u, C.c_float, _f32p, _u, _f32p, _u, C.c_float,
                                 _f32p, _u, _u]
        lib.ref_forward_bias.argtypes = [_u, _f32p, _f32p, _u, _u, _u]
        lib.ref_batchnorm_normalize.argtypes = [_u, _f32p, _f32p, _f32p, _u, _u, _u]
        lib.ref_batchnorm_scale_down.argtypes = [_u, _f32p, _f32p, _u, _u, _u]
        lib.ref_shortcut.argtypes = [_u, _u, _u, _u, _f32p, _u, _u, _u, _f32p, _u]
        lib.ref_activation.argtypes = [_u, _f32p, _u]
        lib.ref_activation.restype = C.c_int
        _ref = lib
    return _ref


class RefNet:
    """A network built from cfg text by the reference's own config parser and layer classes."""

    def __init__(self, cfg_text):
        lib = ref()
        with tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False) as f:
            f.write(cfg_text)
            path = f.name
        self.h = lib.ref_net_create(path.encode())
        os.unlink(path)
        dims = (_u * 3)()
        lib.ref_net_dims(self.h, dims)
        self.batch_size, self.time_step, self.input_size = dims[0], dims[1], dims[2]
        self.n = lib.ref_net_num_layers(self.h)

    def layer_dims(self, i):
        d = (_u * 8)()
        ref().ref_net_layer_dims(self.h, i, d)
        keys = ("layer_type", "activation_type", "output_height", "output_width", "output_channel",
                "output_size", "input_size", "padding")
        return dict(zip(keys, list(d)))

    def load_weights(self, blob):
        with tempfile.NamedTemporaryFile("wb", suffix=".wgh", delete=False) as f:
            f.write(np.asarray(blob, np.float32).tobytes())
            path = f.name
        ref().ref_net_load_weights(self.h, path.encode())
        os.unlink(path)

    def forward(self, x):
        x = _f32(x)
        assert x.size == self.input_size * self.batch_size, (x.size, self.input_size, self.batch_size)
        ref().ref_net_forward(self.h, _fp(x))
        outs = []
        for i in range(self.n):
            d = self.layer_dims(i)
            p = ref().ref_net_output(self.h, i)
            n = d["output_size"] * self.batch_size
            outs.append(np.ctypeslib.as_array(p, shape=(n,)).copy())
        return outs

    def pool_index(self, i):
        d = self.layer_dims(i)
        p = ref().ref_net_pool_index(self.h, i)
        if not p:
            return None
        return np.ctypeslib.as_array(p, shape=(d["output_size"] * self.batch_size,)).copy()
