"""ctypes view of the C ABI in include/nebula_hip.h (nebula_amd/lib/libnebula_hip.so).

This is plumbing for tests, smoke() and bench.py: device buffers, status checking and numpy
conversion.  There is no CPU fallback: a missing library or a failing call raises.
"""
import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
HIP_SO = os.path.join(PKG, "lib", "libnebula_hip.so")

ACT_NAMES = ["undefined_activation", "elu", "hardtan", "leaky", "lhtan", "linear", "loggy", "logistic",
             "plse", "ramp", "relie", "relu", "stair", "tanh"]
ACT = {n: i for i, n in enumerate(ACT_NAMES)}
POOL_MAX, POOL_AVG = 0, 1
LAUNCH_SOURCES = ["none", "pinned", "table", "searched", "model"]      # enum nbl_launch_source

_vp = C.c_void_p
_u = C.c_uint
_f32p = C.POINTER(C.c_float)
_pp = C.POINTER(_f32p)

# name -> (restype, argtypes); also the list of symbols the header declares
SIGNATURES = {
    "nbl_ctx_create": (C.c_int, [C.c_int, C.POINTER(_vp)]),
    "nbl_ctx_create_on_stream": (C.c_int, [C.c_int, _vp, C.POINTER(_vp)]),
    "nbl_ctx_destroy": (C.c_int, [_vp]),
    "nbl_last_error": (C.c_char_p, [_vp]),
    "nbl_ctx_stream": (_vp, [_vp]),
    "nbl_malloc": (C.c_int, [_vp, C.POINTER(_vp), C.c_size_t]),
    "nbl_free": (C.c_int, [_vp, _vp]),
    "nbl_h2d": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "nbl_d2h": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "nbl_d2h_async": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "nbl_malloc_host": (C.c_int, [_vp, C.POINTER(_vp), C.c_size_t]),
    "nbl_free_host": (C.c_int, [_vp, _vp]),
    "nbl_fill_zero": (C.c_int, [_vp, _vp, C.c_size_t]),
    "nbl_copy_d2d": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "nbl_sync": (C.c_int, [_vp]),
    "nbl_lds_fill": (C.c_int, [_vp, _u]),
    "nbl_launch_table_load": (C.c_int, [C.c_char_p]),
    "nbl_launch_table_save": (C.c_int, [C.c_char_p]),
    "nbl_launch_table_clear": (C.c_int, []),
    "nbl_launch_table_size": (C.c_int, []),
    "nbl_launch_table_set_search": (C.c_int, [C.c_int]),
    "nbl_conv2d_plan_launch_source": (C.c_int, [_vp]),
    "nbl_lstm_fwd_tokens": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u, _u]),
    "nbl_rnn_pack": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _u, _u, C.c_int, C.POINTER(_vp)]),
    "nbl_rnn_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u, _u]),
    "nbl_rnn_fwd_tokens": (C.c_int, [_vp, _vp, _vp, _vp, _u, _u]),
    "nbl_rnn_plan_destroy": (C.c_int, [_vp, _vp]),
    "nbl_topk_matches": (C.c_int, [_vp, _vp, _vp, _u, _u, _u, _vp]),
    "nbl_target_prob_sum": (C.c_int, [_vp, _vp, _vp, _u, _u, _vp]),
    "nbl_image_to_input": (C.c_int, [_vp, _vp, _u, _u, _u, _u, _vp, _u, _u]),
    "nbl_conv2d_pack": (C.c_int, [_vp, _f32p, _f32p, _f32p, _f32p, _f32p, _u, _u, _u, _u, _u, _u, _u, C.c_int,
                                  C.POINTER(_vp)]),
    "nbl_conv2d_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u]),
    "nbl_conv2d_shortcut_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u, _u, _u, _vp, _u, C.c_int]),
    "nbl_conv2d_plan_destroy": (C.c_int, [_vp, _vp]),
    "nbl_conv2d_plan_info": (C.c_int, [_vp, C.POINTER(_u), C.POINTER(_u), C.POINTER(C.c_double)]),
    "nbl_conv2d_plan_set_variant": (C.c_int, [_vp, C.c_int]),
    "nbl_conv2d_plan_set_split": (C.c_int, [_vp, C.c_int]),
    "nbl_conv2d_plan_last_launch": (C.c_int, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "nbl_conv2d_num_variants": (C.c_int, []),
    "nbl_conv2d_variant_name": (C.c_char_p, [C.c_int]),
    "nbl_im2col": (C.c_int, [_vp, _vp, _u, _u, _u, _u, _u, _u, _vp]),
    "nbl_fc_pack": (C.c_int, [_vp, _f32p, _f32p, _f32p, _f32p, _f32p, _u, _u, C.c_int, C.POINTER(_vp)]),
    "nbl_fc_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u]),
    "nbl_fc_plan_destroy": (C.c_int, [_vp, _vp]),
    "nbl_fc_plan_set_kernel": (C.c_int, [_vp, C.c_int]),
    "nbl_fc_fwd_noalloc": (C.c_int, [_vp, _vp, _vp, _vp, _u]),
    "nbl_lstm_pack": (C.c_int, [_vp, _pp, _pp, _pp, _pp, _pp, _u, _u, C.c_int, C.POINTER(_vp)]),
    "nbl_lstm_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u, _u]),
    "nbl_lstm_plan_carry_state": (C.c_int, [_vp, _vp, C.c_int]),
    "nbl_lstm_plan_reset_state": (C.c_int, [_vp, _vp]),
    "nbl_lstm_plan_set_state": (C.c_int, [_vp, _vp, _vp, _vp, _u]),
    "nbl_lstm_plan_destroy": (C.c_int, [_vp, _vp]),
    "nbl_pool_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, C.c_int]),
    "nbl_pool_out_dim": (_u, [_u, _u, _u]),
    "nbl_conv_out_dim": (_u, [_u, _u, _u, _u]),
    "nbl_shortcut_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _u, _u, _u, _u, _u, _u, _u, C.c_int]),
    "nbl_softmax_fwd": (C.c_int, [_vp, _vp, _vp, _u, _u]),
    "nbl_activation_fwd": (C.c_int, [_vp, _vp, C.c_size_t, C.c_int]),
    "nbl_forward_bias": (C.c_int, [_vp, _vp, _vp, _u, _u, _u]),
    "nbl_batchnorm_inference": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _u, _u, _u]),
    "nbl_timer_start": (C.c_int, [_vp]),
    "nbl_timer_stop": (C.c_int, [_vp, C.POINTER(C.c_float)]),
    "nbl_version": (C.c_char_p, []),
}

_lib = None


class NebulaHipError(RuntimeError):
    def __init__(self, code, msg):
        RuntimeError.__init__(self, "nebula_hip error %d: %s" % (code, msg))
        self.code = code


def lib():
    """The loaded library.  Raises if it has not been built (python -m nebula_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(HIP_SO):
            raise ImportError("%s is missing: build it with `python -m nebula_amd.build` "
                              "(there is no CPU fallback)" % HIP_SO)
        l = C.CDLL(HIP_SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


class DeviceArray:
    """A device allocation with a shape; freed with the context or by free()."""

    def __init__(self, ctx, shape, dtype=np.float32):
        self.ctx, self.shape, self.dtype = ctx, tuple(int(s) for s in shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = _vp()
        ctx.check(lib().nbl_malloc(ctx.h, C.byref(p), max(self.nbytes, 16)))
        self.ptr = p.value
        ctx._live.append(self)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.shape, self.shape)
        self.ctx.check(lib().nbl_h2d(self.ctx.h, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        self.ctx.check(lib().nbl_d2h(self.ctx.h, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def zero(self):
        self.ctx.check(lib().nbl_fill_zero(self.ctx.h, self.ptr, self.nbytes))
        return self

    def reshape(self, *shape):
        v = DeviceArray.__new__(DeviceArray)
        v.ctx, v.dtype, v.ptr, v.nbytes = self.ctx, self.dtype, self.ptr, self.nbytes
        v.shape = tuple(int(s) for s in (shape[0] if len(shape) == 1 and isinstance(shape[0], (tuple, list)) else shape))
        assert int(np.prod(v.shape, dtype=np.int64)) * v.dtype.itemsize == v.nbytes
        return v

    def free(self):
        if self.ptr:
            self.ctx.check(lib().nbl_free(self.ctx.h, self.ptr))
            self.ptr = None
            if self in self.ctx._live:
                self.ctx._live.remove(self)


class Ctx:
    def __init__(self, device=0):
        h = _vp()
        rc = lib().nbl_ctx_create(device, C.byref(h))
        if rc != 0:
            raise NebulaHipError(rc, lib().nbl_last_error(None).decode())
        self.h = h
        self._live = []
        self._plans = []

    def check(self, rc):
        if rc != 0:
            raise NebulaHipError(rc, lib().nbl_last_error(self.h).decode())

    def close(self):
        if self.h:
            for kind, p in self._plans:
                getattr(lib(), "nbl_%s_plan_destroy" % kind)(self.h, p)
            self._plans = []
            for a in list(self._live):
                a.free()
            lib().nbl_ctx_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- memory ----
    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def array(self, a, dtype=np.float32):
        a = np.ascontiguousarray(a, dtype=dtype)
        return DeviceArray(self, a.shape, dtype).upload(a)

    def sync(self):
        self.check(lib().nbl_sync(self.h))

    def target_prob_sum(self, probs, targets):
        """sum_r probs[r][targets[r]] (probs: DeviceArray [rows][n] float32, targets: DeviceArray [rows] uint32)."""
        rows, n = probs.shape
        out = self.empty((1,))
        self.check(lib().nbl_target_prob_sum(self.h, probs.ptr, targets.ptr, rows, n, out.ptr))
        v = float(out.numpy()[0])
        out.free()
        return v

    def image_to_input(self, images_u8, dst_h, dst_w):
        """images_u8: DeviceArray [n][h][w][c] of uint8 -> DeviceArray [n][c][dst_h][dst_w] of float32."""
        n, h, w, c = images_u8.shape
        out = self.empty((n, c, dst_h, dst_w))
        self.check(lib().nbl_image_to_input(self.h, images_u8.ptr, n, h, w, c, out.ptr, dst_h, dst_w))
        return out

    def copy(self, dst, src, nbytes=None):
        """Device-to-device copy kernel between two DeviceArrays."""
        n = src.nbytes if nbytes is None else nbytes
        assert n <= dst.nbytes and n <= src.nbytes
        self.check(lib().nbl_copy_d2d(self.h, dst.ptr, src.ptr, n))

    def timer_start(self):
        self.check(lib().nbl_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        self.check(lib().nbl_timer_stop(self.h, C.byref(ms)))
        return ms.value

    # ---- plans ----
    def conv_pack(self, weight, bias, bn=None, H=None, W=None, stride=1, pad=0, act="linear"):
        weight, bias = _f32(weight), _f32(bias)
        F, Cc, k, _ = weight.shape
        sc, mu, var = (None, None, None) if bn is None else [_f32(a) for a in bn]
        p = _vp()
        self.check(lib().nbl_conv2d_pack(self.h, _fp(weight), _fp(bias), _fp(sc), _fp(mu), _fp(var), Cc, H, W, F, k,
                                         stride, pad, ACT[act], C.byref(p)))
        self._plans.append(("conv2d", p))
        return ConvPlan(self, p, Cc, H, W, F)

    def fc_pack(self, weight, bias, bn=None, act="linear"):
        weight, bias = _f32(weight), _f32(bias)
        O, I = weight.shape
        sc, mu, var = (None, None, None) if bn is None else [_f32(a) for a in bn]
        p = _vp()
        self.check(lib().nbl_fc_pack(self.h, _fp(weight), _fp(bias), _fp(sc), _fp(mu), _fp(var), I, O, ACT[act],
                                     C.byref(p)))
        self._plans.append(("fc", p))
        return FcPlan(self, p, I, O)

    def lstm_pack(self, weight, bias, bn=None, act="linear"):
        """weight/bias: 8 arrays in file order iW,fW,oW,cW,iU,fU,oU,cU; bn = (scale8, mean8, var8)."""
        weight = [_f32(w) for w in weight]
        bias = [_f32(b) for b in bias]
        H, I = weight[4].shape

        def arr(xs):
            return None if xs is None else (_f32p * 8)(*[_fp(a) for a in xs])
        keep = [weight, bias]
        if bn is not None:
            bn = [[_f32(a) for a in grp] for grp in bn]
            keep.append(bn)
        sc, mu, var = (None, None, None) if bn is None else bn
        p = _vp()
        self.check(lib().nbl_lstm_pack(self.h, arr(weight), arr(bias), arr(sc), arr(mu), arr(var), I, H, ACT[act],
                                       C.byref(p)))
        self._plans.append(("lstm", p))
        return LstmPlan(self, p, I, H)

    def rnn_pack(self, weight, bias, bn=None, act="linear"):
        """weight/bias: 3 arrays in file order input, hidden, output gate; bn = (scale3, mean3, var3)."""
        weight = [_f32(w) for w in weight]
        bias = [_f32(b) for b in bias]
        O, I = weight[0].shape

        def arr(xs):
            return None if xs is None else (_f32p * 3)(*[_fp(a) for a in xs])
        if bn is not None:
            bn = [[_f32(a) for a in grp] for grp in bn]
        sc, mu, var = (None, None, None) if bn is None else bn
        p = _vp()
        self.check(lib().nbl_rnn_pack(self.h, arr(weight), arr(bias), arr(sc), arr(mu), arr(var), I, O, ACT[act],
                                      C.byref(p)))
        self._plans.append(("rnn", p))
        return RnnPlan(self, p, I, O)

    def topk_matches(self, probs, labels, k):
        """rows of probs (DeviceArray [rows][n]) whose label (DeviceArray [rows] uint32) is among the k largest."""
        rows, n = probs.shape
        out = self.empty((4,), np.uint32)
        self.check(lib().nbl_topk_matches(self.h, probs.ptr, labels.ptr, rows, n, k, out.ptr))
        v = int(out.numpy()[0])
        out.free()
        return v

    # ---- one-shot ops on DeviceArrays ----
    def im2col(self, x, k, s, p):
        Cc, H, W = x.shape
        oh, ow = lib().nbl_conv_out_dim(H, k, s, p), lib().nbl_conv_out_dim(W, k, s, p)
        col = self.empty((Cc * k * k, oh * ow))
        self.check(lib().nbl_im2col(self.h, x.ptr, Cc, H, W, k, s, p, col.ptr))
        return col

    def pool(self, x, k, s, p, mode="max", want_index=True):
        B, Cc, H, W = x.shape
        oh, ow = lib().nbl_pool_out_dim(H, s, p), lib().nbl_pool_out_dim(W, s, p)
        y = self.empty((B, Cc, oh, ow))
        idx = self.empty((B, Cc, oh, ow), np.uint32) if (mode == "max" and want_index) else None
        self.check(lib().nbl_pool_fwd(self.h, x.ptr, y.ptr, idx.ptr if idx is not None else None, B, Cc, H, W, k, s, p,
                                      POOL_MAX if mode == "max" else POOL_AVG))
        return (y, idx) if mode == "max" else y

    def shortcut(self, prev, conn, act="linear", out=None):
        B, oc, oh, ow = prev.shape
        _, ic, ih, iw = conn.shape
        y = out if out is not None else self.empty(prev.shape)
        self.check(lib().nbl_shortcut_fwd(self.h, prev.ptr, conn.ptr, y.ptr, B, ic, ih, iw, oc, oh, ow, ACT[act]))
        return y

    def softmax(self, x):
        rows, n = x.shape[0], int(np.prod(x.shape[1:]))
        y = self.empty((rows, n))
        self.check(lib().nbl_softmax_fwd(self.h, x.ptr, y.ptr, rows, n))
        return y

    def activation(self, x, act):
        self.check(lib().nbl_activation_fwd(self.h, x.ptr, x.size, ACT[act] if isinstance(act, str) else act))
        return x

    def forward_bias(self, y, bias, channel, size, batch):
        self.check(lib().nbl_forward_bias(self.h, y.ptr, bias.ptr, channel, size, batch))
        return y

    def batchnorm_inference(self, y, mean, var, scale, channel, size, batch):
        self.check(lib().nbl_batchnorm_inference(self.h, y.ptr, mean.ptr, var.ptr, scale.ptr, channel, size, batch))
        return y


class ConvPlan:
    def __init__(self, ctx, p, Cc, H, W, F):
        self.ctx, self.p, self.C, self.H, self.W, self.F = ctx, p, Cc, H, W, F
        oh, ow, fl = _u(), _u(), C.c_double()
        ctx.check(lib().nbl_conv2d_plan_info(p, C.byref(oh), C.byref(ow), C.byref(fl)))
        self.OH, self.OW, self.flop_per_image = oh.value, ow.value, fl.value

    def set_variant(self, v):
        self.ctx.check(lib().nbl_conv2d_plan_set_variant(self.p, v))

    def last_launch(self):
        """(tile shape index, k slices) of the most recent launch."""
        v, g = C.c_int(), C.c_int()
        self.ctx.check(lib().nbl_conv2d_plan_last_launch(self.p, C.byref(v), C.byref(g)))
        return v.value, g.value

    def launch_source(self):
        return LAUNCH_SOURCES[lib().nbl_conv2d_plan_launch_source(self.p)]

    def set_split(self, mode):
        """-1: measured on first use, 0: never split along k, 1: split wherever the cost model says so, 2..8: that many slices."""
        self.ctx.check(lib().nbl_conv2d_plan_set_split(self.p, mode))

    def __call__(self, x, out=None):
        B = x.shape[0]
        y = out if out is not None else self.ctx.empty((B, self.F, self.OH, self.OW))
        self.ctx.check(lib().nbl_conv2d_fwd(self.ctx.h, self.p, x.ptr, y.ptr, B))
        return y


    def with_shortcut(self, x, conn, post_act="linear", out=None):
        B = x.shape[0]
        _, cc, ch, cw = conn.shape
        y = out if out is not None else self.ctx.empty((B, self.F, self.OH, self.OW))
        self.ctx.check(lib().nbl_conv2d_shortcut_fwd(self.ctx.h, self.p, x.ptr, conn.ptr, cc, ch, cw, y.ptr, B, ACT[post_act]))
        return y


class FcPlan:
    def __init__(self, ctx, p, I, O):
        self.ctx, self.p, self.I, self.O = ctx, p, I, O

    def __call__(self, x, out=None):
        B = x.shape[0]
        assert x.size == B * self.I
        y = out if out is not None else self.ctx.empty((B, self.O))
        self.ctx.check(lib().nbl_fc_fwd(self.ctx.h, self.p, x.ptr, y.ptr, B))
        return y

    def set_kernel(self, kind):
        """0: chosen by shape, 1: the LDS-tiled kernels, 2: the weight-streaming kernel wherever it applies."""
        self.ctx.check(lib().nbl_fc_plan_set_kernel(self.p, kind))

    def noalloc(self, x, out):
        """The same product through the entry point that allocates nothing (static device scratch)."""
        B = x.shape[0]
        assert x.size == B * self.I and out.size == B * self.O
        self.ctx.check(lib().nbl_fc_fwd_noalloc(self.ctx.h, self.p, x.ptr, out.ptr, B))
        return out


class RnnPlan:
    def __init__(self, ctx, p, I, O):
        self.ctx, self.p, self.I, self.O = ctx, p, I, O

    def __call__(self, x, out=None):
        T, B, I = x.shape
        assert I == self.I
        y = out if out is not None else self.ctx.empty((T, B, self.O))
        self.ctx.check(lib().nbl_rnn_fwd(self.ctx.h, self.p, x.ptr, y.ptr, T, B))
        return y


class LstmPlan:
    def __init__(self, ctx, p, I, H):
        self.ctx, self.p, self.I, self.H = ctx, p, I, H

    def __call__(self, x, out=None, cell=None):
        T, B, I = x.shape
        assert I == self.I
        y = out if out is not None else self.ctx.empty((T, B, self.H))
        self.ctx.check(lib().nbl_lstm_fwd(self.ctx.h, self.p, x.ptr, y.ptr, cell.ptr if cell is not None else None, T, B))
        return y

    def carry_state(self, on=True):
        """Start every pass from the state the previous pass of the same batch size ended with (off: from zero)."""
        self.ctx.check(lib().nbl_lstm_plan_carry_state(self.ctx.h, self.p, 1 if on else 0))

    def reset_state(self):
        self.ctx.check(lib().nbl_lstm_plan_reset_state(self.ctx.h, self.p))

    def set_state(self, h, c):
        """h, c: DeviceArrays [B][H], the state the next pass of that batch size starts from."""
        self.ctx.check(lib().nbl_lstm_plan_set_state(self.ctx.h, self.p, h.ptr, c.ptr, h.shape[0]))

    def from_tokens(self, tokens, out=None, cell=None):
        """tokens: DeviceArray [T][B] of uint32, the positions of the 1s of one-hot input rows."""
        T, B = tokens.shape
        y = out if out is not None else self.ctx.empty((T, B, self.H))
        self.ctx.check(lib().nbl_lstm_fwd_tokens(self.ctx.h, self.p, tokens.ptr, y.ptr,
                                                 cell.ptr if cell is not None else None, T, B))
        return y
