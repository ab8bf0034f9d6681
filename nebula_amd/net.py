"""ctypes view of include/nebula_layers.h (nebula_amd/lib/libnebula_layers.so): cfg-driven networks
built from the C++ layer classes.  Plumbing for tests, smoke() and bench.py; no CPU fallback."""
import ctypes as C
import os

import numpy as np

from . import hip

LAYERS_SO = os.path.join(hip.PKG, "lib", "libnebula_layers.so")

LAYER_TYPES = ["undefined_layer", "connected_layer", "convolutional_layer", "cost_layer", "dropout_layer",
               "avgpool_layer", "maxpool_layer", "shortcut_layer", "softmax_layer", "rnn_layer", "lstm_layer",
               "rbm_layer"]

_vp, _u = C.c_void_p, C.c_uint
SIGNATURES = {
    "nbl_net_create": (C.c_int, [C.c_char_p, C.c_int, _u, C.c_int, C.c_char_p, C.POINTER(_vp)]),
    "nbl_net_destroy": (C.c_int, [_vp]),
    "nbl_net_last_error": (C.c_char_p, []),
    "nbl_net_load_weights": (C.c_int, [_vp, C.c_char_p]),
    "nbl_net_store_weights": (C.c_int, [_vp, C.c_char_p]),
    "nbl_net_weight_layout": (C.c_int, [_vp, C.POINTER(_u), C.c_size_t, C.POINTER(C.c_size_t)]),
    "nbl_net_dims": (C.c_int, [_vp, C.POINTER(_u)]),
    "nbl_net_num_layers": (C.c_int, [_vp]),
    "nbl_net_layer_info": (C.c_int, [_vp, C.c_int, C.POINTER(_u)]),
    "nbl_net_layer_flop": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_double)]),
    "nbl_net_set_input": (C.c_int, [_vp, _vp, C.c_size_t]),
    "nbl_net_set_input_images": (C.c_int, [_vp, _vp, _u, _u, _u]),
    "nbl_net_set_input_tokens": (C.c_int, [_vp, _vp, C.c_size_t]),
    "nbl_net_accumulate_perplexity": (C.c_int, [_vp, _vp, C.c_size_t, C.POINTER(C.c_float)]),
    "nbl_net_accumulate_topk": (C.c_int, [_vp, _vp, C.c_size_t, _u, C.POINTER(_u)]),
    "nbl_net_forward": (C.c_int, [_vp]),
    "nbl_net_sync": (C.c_int, [_vp]),
    "nbl_net_forward_timed": (C.c_int, [_vp, C.POINTER(C.c_float)]),
    "nbl_net_layer_output": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t]),
    "nbl_net_layer_output_writer": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_int)]),
    "nbl_net_pool_index": (C.c_int, [_vp, C.c_int, _vp, C.c_size_t]),
    "nbl_net_conv_last_launch": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "nbl_net_conv_pin_launch": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int]),
    "nbl_net_conv_launch_source": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_int)]),
    "nbl_net_conv_problem": (C.c_int, [_vp, C.c_int, C.POINTER(_u)]),
    "nbl_net_softmax_copy": (C.c_int, [_vp, C.c_int]),
    "nbl_net_set_graph": (C.c_int, [_vp, C.c_int]),
    "nbl_net_set_carry_state": (C.c_int, [_vp, C.c_int]),
    "nbl_net_reset_state": (C.c_int, [_vp]),
    "nbl_net_graph_active": (C.c_int, [_vp]),
    "nbl_net_ctx": (_vp, [_vp]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        hip.lib()     # dependency, and the loud failure if nothing is built
        if not os.path.exists(LAYERS_SO):
            raise ImportError("%s is missing: build it with `python -m nebula_amd.build`" % LAYERS_SO)
        l = C.CDLL(LAYERS_SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


class NetworkError(RuntimeError):
    pass


class Network:
    """A cfg-described network on the GPU."""

    def __init__(self, cfg, is_text=True, batch=0, device=0, weights=None):
        h = _vp()
        rc = lib().nbl_net_create(cfg.encode(), 1 if is_text else 0, batch, device,
                                  weights.encode() if weights else None, C.byref(h))
        if rc != 0:
            raise NetworkError(lib().nbl_net_last_error().decode())
        self.h = h
        d = (_u * 6)()
        lib().nbl_net_dims(self.h, d)
        self.batch_size, self.time_step, self.input_size = d[0], d[1], d[2]
        self.input_shape = (d[5], d[3], d[4])
        self.num_layers = lib().nbl_net_num_layers(self.h)

    def _check(self, rc):
        if rc != 0:
            raise NetworkError(lib().nbl_net_last_error().decode())

    def close(self):
        if self.h:
            lib().nbl_net_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def load_weights(self, path):
        self._check(lib().nbl_net_load_weights(self.h, path.encode()))

    def load_weight_blob(self, blob):
        import tempfile
        with tempfile.NamedTemporaryFile("wb", suffix=".wgh", delete=False) as f:
            f.write(np.ascontiguousarray(blob, np.float32).tobytes())
            path = f.name
        try:
            self.load_weights(path)
        finally:
            os.unlink(path)

    def weight_layout(self):
        """[(layer index, kind, count, fan_in)] in .wgh order; kind in bias/weight/scale/mean/var."""
        n = C.c_size_t()
        self._check(lib().nbl_net_weight_layout(self.h, None, 0, C.byref(n)))
        buf = (_u * (4 * n.value))()
        self._check(lib().nbl_net_weight_layout(self.h, buf, n.value, C.byref(n)))
        names = ("bias", "weight", "scale", "mean", "var")
        return [(buf[4 * i], names[buf[4 * i + 1]], buf[4 * i + 2], buf[4 * i + 3]) for i in range(n.value)]

    def layer_info(self, i):
        d = (_u * 8)()
        self._check(lib().nbl_net_layer_info(self.h, i, d))
        keys = ("layer_type", "activation_type", "output_channel", "output_height", "output_width", "output_size",
                "input_size", "padding")
        out = dict(zip(keys, list(d)))
        out["kind"] = LAYER_TYPES[out["layer_type"]]
        return out

    def layer_flop(self, i):
        f = C.c_double()
        self._check(lib().nbl_net_layer_flop(self.h, i, C.byref(f)))
        return f.value

    def set_input(self, x):
        x = np.ascontiguousarray(x, np.float32)
        self._check(lib().nbl_net_set_input(self.h, x.ctypes.data, x.size))

    def set_input_images(self, images_u8):
        """uint8 [batch][height][width][channels], decoded channel order (B, G, R)."""
        a = np.ascontiguousarray(images_u8, np.uint8)
        n, h, w, _ = a.shape
        self._check(lib().nbl_net_set_input_images(self.h, a.ctypes.data, n, h, w))

    def set_input_tokens(self, tokens):
        """uint32 [time_steps][sequences]: index of the 1 of every one-hot input row."""
        t = np.ascontiguousarray(tokens, np.uint32)
        self._check(lib().nbl_net_set_input_tokens(self.h, t.ctypes.data, t.size))

    def accumulate_perplexity(self, label_tokens):
        t = np.ascontiguousarray(label_tokens, np.uint32)
        out = C.c_float()
        self._check(lib().nbl_net_accumulate_perplexity(self.h, t.ctypes.data, t.size, C.byref(out)))
        return out.value

    def accumulate_topk(self, labels, k):
        t = np.ascontiguousarray(labels, np.uint32)
        out = _u()
        self._check(lib().nbl_net_accumulate_topk(self.h, t.ctypes.data, t.size, k, C.byref(out)))
        return out.value

    def forward(self):
        self._check(lib().nbl_net_forward(self.h))

    def sync(self):
        self._check(lib().nbl_net_sync(self.h))

    def forward_timed(self):
        ms = (C.c_float * self.num_layers)()
        self._check(lib().nbl_net_forward_timed(self.h, ms))
        return list(ms)

    def output(self, i):
        info = self.layer_info(i)
        out = np.empty(info["output_size"] * self.batch_size, np.float32)
        self._check(lib().nbl_net_layer_output(self.h, i, out.ctypes.data, out.size))
        return out

    def output_writer(self, i):
        """Index of the layer whose values output(i) returns (i itself unless the tensor is shared or overwritten)."""
        w = C.c_int()
        self._check(lib().nbl_net_layer_output_writer(self.h, i, C.byref(w)))
        return w.value

    def pool_index(self, i):
        info = self.layer_info(i)
        out = np.empty(info["output_size"] * self.batch_size, np.uint32)
        self._check(lib().nbl_net_pool_index(self.h, i, out.ctypes.data, out.size))
        return out

    def conv_last_launch(self, i):
        """(tile shape index, k slices) of convolutional layer i's most recent launch."""
        v, g = C.c_int(), C.c_int()
        self._check(lib().nbl_net_conv_last_launch(self.h, i, C.byref(v), C.byref(g)))
        return v.value, g.value

    def conv_problem(self, i):
        """Launch-table key of convolutional layer i: (C, H, W, F, size, stride, padding, batch, res_c, res_h, res_w, in_place)."""
        key = (_u * 12)()
        self._check(lib().nbl_net_conv_problem(self.h, i, key))
        return tuple(key)

    def conv_launch_source(self, i):
        """Where layer i's most recent launch took its tile shape from: one of hip.LAUNCH_SOURCES."""
        v = C.c_int()
        self._check(lib().nbl_net_conv_launch_source(self.h, i, C.byref(v)))
        return hip.LAUNCH_SOURCES[v.value]

    def conv_pin_launch(self, i, variant, split):
        """Pin layer i's tile shape (variant < 0: searched) and k-split (-1 searched, 0 never, 1 cost model, 2..8 slices)."""
        self._check(lib().nbl_net_conv_pin_launch(self.h, i, variant, split))

    def softmax_copy(self, enabled):
        lib().nbl_net_softmax_copy(self.h, 1 if enabled else 0)

    def set_graph(self, enabled):
        """Record one forward pass into a HIP graph and replay it from then on (first pass eager, second recorded)."""
        lib().nbl_net_set_graph(self.h, 1 if enabled else 0)

    def set_carry_state(self, enabled):
        """[lstm] layers start a pass from the state their previous pass ended with (also [net] carry_state=1)."""
        self._check(lib().nbl_net_set_carry_state(self.h, 1 if enabled else 0))

    def reset_state(self):
        """The next pass of a carrying network starts from zero state again (a new token stream)."""
        self._check(lib().nbl_net_reset_state(self.h))

    @property
    def graph_active(self):
        return lib().nbl_net_graph_active(self.h) == 1

    @property
    def ctx(self):
        return lib().nbl_net_ctx(self.h)

    def timer_start(self):
        rc = hip.lib().nbl_timer_start(self.ctx)
        if rc != 0:
            raise NetworkError("nbl_timer_start failed")

    def timer_stop(self):
        ms = C.c_float()
        rc = hip.lib().nbl_timer_stop(self.ctx, C.byref(ms))
        if rc != 0:
            raise NetworkError("nbl_timer_stop failed")
        return ms.value
