"""TEST INFRASTRUCTURE: ctypes loaders for the two CPU checkers.

* ``Oracle``  -- oracle/libotter_int8_oracle.so, the repo's own C restatement (always buildable with gcc).
* ``Ref``     -- oracle/_ref/libotter_ref.so, the real reference compiled from /root/reference by
                 oracle/Makefile (present only where that build ran; travels to the GPU box as a built file).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
All arrays are NCHW numpy arrays (int8 / int32 / float32).
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libotter_int8_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libotter_ref.so")
# the same reference plus the reference-side binding of the GPU library (oracle/ref_hip_layer.cpp)
REF_HIP_SO = os.path.join(HERE, "_ref", "libotter_ref_hip.so")

ROUND_SSE, ROUND_EXACT = 0, 1

_f32p = C.POINTER(C.c_float)
_i8p = C.POINTER(C.c_int8)
_i32p = C.POINTER(C.c_int32)


def _p(a, typ):
    if a is None:
        return C.cast(None, typ)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(typ)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def build_oracle():
    subprocess.check_call(["make", "-C", HERE, "oracle"], stdout=subprocess.DEVNULL)


def build_ref(jobs=8):
    subprocess.check_call(["make", "-C", HERE, "-j%d" % jobs, "ref"], stdout=subprocess.DEVNULL)


def out_size(i, k, s, p, d=1):
    return (i + 2 * p - d * (k - 1) - 1) // s + 1


class Oracle:
    def __init__(self):
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        L = self.lib = C.CDLL(ORACLE_SO)
        L.otter_oracle_float2int8.restype = C.c_int8
        L.otter_oracle_float2int8.argtypes = [C.c_float, C.c_int]
        L.otter_oracle_activation.restype = C.c_float
        L.otter_oracle_activation.argtypes = [C.c_float, C.c_int, _f32p]
        L.otter_oracle_conv_int32.restype = C.c_int
        L.otter_oracle_conv_layer_forward.restype = C.c_int
        L.otter_oracle_num_threads.restype = C.c_int

    def set_num_threads(self, n):
        self.lib.otter_oracle_set_num_threads(C.c_int(n))

    def num_threads(self):
        return self.lib.otter_oracle_num_threads()

    def float2int8(self, v, mode):
        return int(self.lib.otter_oracle_float2int8(C.c_float(v), mode))

    def quantize_round_mode(self, c, use_packing=True):
        return self.lib.otter_oracle_quantize_round_mode(C.c_int(c), C.c_int(int(use_packing)))

    def requantize_round_mode(self, c, k, groups, use_packing=True):
        return self.lib.otter_oracle_requantize_round_mode(C.c_int(c), C.c_int(k), C.c_int(groups),
                                                           C.c_int(int(use_packing)))

    def scale_in(self, weight_scales, in_scale):
        ws = _f32(weight_scales)
        out = np.empty_like(ws)
        self.lib.otter_oracle_scale_in(_p(ws, _f32p), C.c_int(ws.size), C.c_float(in_scale), _p(out, _f32p))
        return out

    def quantize(self, x, scales, mode):
        x = _f32(x)
        n, c, h, w = x.shape
        s = _f32(np.atleast_1d(scales))
        out = np.empty(x.shape, np.int8)
        self.lib.otter_oracle_quantize(_p(x, _f32p), n, c, h, w, _p(s, _f32p), C.c_int(s.size), C.c_int(mode),
                                       _p(out, _i8p))
        return out

    def conv_int32(self, xq, wq, stride=(1, 1), pad=(0, 0), dil=(1, 1), groups=1):
        xq = np.ascontiguousarray(xq, np.int8)
        wq = np.ascontiguousarray(wq, np.int8)
        n, c, h, w = xq.shape
        k, cg, kh, kw = wq.shape
        assert cg * groups == c
        oh, ow = out_size(h, kh, stride[0], pad[0], dil[0]), out_size(w, kw, stride[1], pad[1], dil[1])
        out = np.empty((n, k, oh, ow), np.int32)
        rc = self.lib.otter_oracle_conv_int32(_p(xq, _i8p), n, c, h, w, _p(wq, _i8p), k, kh, kw, stride[0], stride[1],
                                              pad[0], pad[1], dil[0], dil[1], groups, _p(out, _i32p))
        if rc != 0:
            raise ValueError("oracle conv rejected the shape")
        return out

    def dequantize(self, acc, scale, bias=None):
        acc = np.ascontiguousarray(acc, np.int32)
        n, c, h, w = acc.shape
        s, b = _f32(np.atleast_1d(scale)), _f32(bias)
        out = np.empty(acc.shape, np.float32)
        self.lib.otter_oracle_dequantize(_p(acc, _i32p), n, c, h * w, _p(s, _f32p), C.c_int(s.size), _p(b, _f32p),
                                         C.c_int(0 if b is None else b.size), _p(out, _f32p))
        return out

    def requantize(self, acc, scale_in, scale_out, bias, act_type, act_params, mode):
        acc = np.ascontiguousarray(acc, np.int32)
        n, c, h, w = acc.shape
        si, so, b = _f32(np.atleast_1d(scale_in)), _f32(np.atleast_1d(scale_out)), _f32(bias)
        ap = _f32(act_params)
        out = np.empty(acc.shape, np.int8)
        self.lib.otter_oracle_requantize(_p(acc, _i32p), n, c, h * w, _p(si, _f32p), C.c_int(si.size),
                                         _p(so, _f32p), C.c_int(so.size), _p(b, _f32p),
                                         C.c_int(0 if b is None else b.size), C.c_int(act_type), _p(ap, _f32p),
                                         C.c_int(mode), _p(out, _i8p))
        return out

    def activation_f32(self, x, act_type, act_params=None):
        x = np.array(x, np.float32, copy=True, order="C")
        ap = _f32(act_params)
        self.lib.otter_oracle_activation_f32(_p(x, _f32p), C.c_size_t(x.size), C.c_int(act_type), _p(ap, _f32p))
        return x

    def conv_layer_forward(self, x, wq, weight_scales, in_scale, *, stride=(1, 1), pad=(0, 0), dil=(1, 1), groups=1,
                           bias=None, top_scale=1.0, int8_out=False, act_type=0, act_params=None, use_packing=True,
                           want_acc=False):
        in_is_int8 = x.dtype == np.int8
        x = np.ascontiguousarray(x, np.int8 if in_is_int8 else np.float32)
        wq = np.ascontiguousarray(wq, np.int8)
        n, c, h, w = x.shape
        k, cg, kh, kw = wq.shape
        oh, ow = out_size(h, kh, stride[0], pad[0], dil[0]), out_size(w, kw, stride[1], pad[1], dil[1])
        ws, b, ap = _f32(np.atleast_1d(weight_scales)), _f32(bias), _f32(act_params)
        out = np.empty((n, k, oh, ow), np.int8 if int8_out else np.float32)
        acc = np.empty((n, k, oh, ow), np.int32) if want_acc else None
        rc = self.lib.otter_oracle_conv_layer_forward(
            x.ctypes.data_as(C.c_void_p), C.c_int(int(in_is_int8)), n, c, h, w, _p(wq, _i8p), k, kh, kw, stride[0],
            stride[1], pad[0], pad[1], dil[0], dil[1], groups, _p(b, _f32p), _p(ws, _f32p), C.c_int(ws.size),
            C.c_float(in_scale), C.c_float(top_scale), C.c_int(int(int8_out)), C.c_int(act_type), _p(ap, _f32p),
            C.c_int(int(use_packing)), _p(acc, _i32p), out.ctypes.data_as(C.c_void_p))
        if rc != 0:
            raise ValueError("oracle conv layer rejected the shape")
        return (out, acc) if want_acc else out

    def pack(self, a, p):
        a = np.ascontiguousarray(a)
        n, c, h, w = a.shape
        assert c % p == 0
        out = np.empty((n, c // p, h, w, p), a.dtype)
        self.lib.otter_oracle_pack(a.ctypes.data_as(C.c_void_p), C.c_size_t(a.itemsize), n, c, h * w, p,
                                   out.ctypes.data_as(C.c_void_p))
        return out

    def unpack(self, a):
        a = np.ascontiguousarray(a)
        n, cp, h, w, p = a.shape
        out = np.empty((n, cp * p, h, w), a.dtype)
        self.lib.otter_oracle_unpack(a.ctypes.data_as(C.c_void_p), C.c_size_t(a.itemsize), n, cp * p, h * w, p,
                                     out.ctypes.data_as(C.c_void_p))
        return out

    def eltwise_add(self, a, b):
        a, b = _f32(a), _f32(b)
        out = np.empty_like(a)
        self.lib.otter_oracle_eltwise_add(_p(a, _f32p), _p(b, _f32p), C.c_size_t(a.size), _p(out, _f32p))
        return out

    def global_avgpool(self, x):
        x = _f32(x)
        n, c, h, w = x.shape
        out = np.empty((n, c), np.float32)
        self.lib.otter_oracle_global_avgpool(_p(x, _f32p), n, c, h * w, _p(out, _f32p))
        return out

    def inner_product(self, x, wt, bias):
        x, wt, bias = _f32(x), _f32(wt), _f32(bias)
        n, in_f = x.shape
        out_f = wt.shape[0]
        out = np.empty((n, out_f), np.float32)
        self.lib.otter_oracle_inner_product(_p(x, _f32p), n, in_f, _p(wt, _f32p), _p(bias, _f32p), out_f,
                                            _p(out, _f32p))
        return out


def ref_available():
    return os.path.exists(REF_SO)


def ref_hip_available():
    return os.path.exists(REF_HIP_SO)


class Ref:
    """The compiled reference. Raises OSError if oracle/_ref/libotter_ref.so is absent or cannot load.
    hip=True: the build that also holds the GPU convolution layer written against the reference's headers
    (use_hip_convolution switches the reference's layer registry to it and back)."""

    def __init__(self, hip=False):
        L = self.lib = C.CDLL(REF_HIP_SO if hip else REF_SO)
        self.hip = hip
        L.otter_ref_last_error.restype = C.c_char_p
        L.otter_ref_conv_layer_create.restype = C.c_void_p
        L.otter_ref_conv_layer_forward.restype = C.c_double
        L.otter_ref_num_threads.restype = C.c_int

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError("reference: " + self.lib.otter_ref_last_error().decode(errors="replace"))

    def num_threads(self):
        return self.lib.otter_ref_num_threads()

    def use_hip_convolution(self, on):
        """Registers the GPU layer under "Convolution" in the reference's LayerRegistry (nets opened afterwards get
        it), or restores the stock creator."""
        assert self.hip
        rc = self.lib.otter_ref_use_hip_convolution(C.c_int(int(on)))
        if rc != 0:
            self.lib.otter_ref_hip_last_error.restype = C.c_char_p
            raise RuntimeError("GPU layer: " + self.lib.otter_ref_hip_last_error().decode(errors="replace"))

    def hip_forward_count(self):
        self.lib.otter_ref_hip_forward_count.restype = C.c_long
        return self.lib.otter_ref_hip_forward_count()

    def set_num_threads(self, n):
        self.lib.otter_ref_set_num_threads(C.c_int(n))

    def quantize(self, x, scales, packing=True):
        x = _f32(x)
        n, c, h, w = x.shape
        s = _f32(np.atleast_1d(scales))
        out = np.empty(x.shape, np.int8)
        self._check(self.lib.otter_ref_quantize(_p(x, _f32p), n, c, h, w, _p(s, _f32p), C.c_int(s.size),
                                                C.c_int(int(packing)), _p(out, _i8p)))
        return out

    def conv_int32(self, xq, wq, stride=(1, 1), pad=(0, 0), dil=(1, 1), groups=1, packing=True):
        xq = np.ascontiguousarray(xq, np.int8)
        wq = np.ascontiguousarray(wq, np.int8)
        n, c, h, w = xq.shape
        k, cg, kh, kw = wq.shape
        oh, ow = out_size(h, kh, stride[0], pad[0], dil[0]), out_size(w, kw, stride[1], pad[1], dil[1])
        out = np.empty((n, k, oh, ow), np.int32)
        self._check(self.lib.otter_ref_conv_int32(_p(xq, _i8p), n, c, h, w, _p(wq, _i8p), k, kh, kw, stride[0],
                                                  stride[1], pad[0], pad[1], dil[0], dil[1], groups,
                                                  C.c_int(int(packing)), _p(out, _i32p), oh, ow))
        return out

    def dequantize(self, acc, scale, bias=None, packing=True):
        acc = np.ascontiguousarray(acc, np.int32)
        n, c, h, w = acc.shape
        s, b = _f32(np.atleast_1d(scale)), _f32(bias)
        out = np.empty(acc.shape, np.float32)
        self._check(self.lib.otter_ref_dequantize(_p(acc, _i32p), n, c, h, w, _p(s, _f32p), C.c_int(s.size),
                                                  _p(b, _f32p), C.c_int(0 if b is None else b.size),
                                                  C.c_int(int(packing)), _p(out, _f32p)))
        return out

    def requantize(self, acc, scale_in, scale_out, bias, act_type, act_params=None, packing=True):
        acc = np.ascontiguousarray(acc, np.int32)
        n, c, h, w = acc.shape
        si, so, b = _f32(np.atleast_1d(scale_in)), _f32(np.atleast_1d(scale_out)), _f32(bias)
        ap = _f32(act_params)
        out = np.empty(acc.shape, np.int8)
        self._check(self.lib.otter_ref_requantize(_p(acc, _i32p), n, c, h, w, _p(si, _f32p), C.c_int(si.size),
                                                  _p(so, _f32p), C.c_int(so.size), _p(b, _f32p),
                                                  C.c_int(0 if b is None else b.size), C.c_int(act_type),
                                                  _p(ap, _f32p), C.c_int(0 if ap is None else ap.size),
                                                  C.c_int(int(packing)), _p(out, _i8p)))
        return out

    # ---- model files and whole networks (Tensor/Otter.cpp, Tensor/Initializer.cpp, Tensor/Net.cpp) ----
    def otter_dump(self, path):
        """The reference's parse of a `.otter` file: 'N name', 'G key=value', 'T block', 'P key=value' lines."""
        self.lib.otter_ref_otter_dump.restype = C.c_long
        buf = C.create_string_buffer(1 << 24)
        n = self.lib.otter_ref_otter_dump(os.fsencode(path), buf, C.c_size_t(len(buf)))
        self._check(0 if n >= 0 else -1)
        return buf.raw[:n].decode(errors="surrogateescape")

    @property
    def ncnn_read_entry(self):
        """(function, error function) of the reference's `.bin` reader, same signature as the host library's."""
        return self.lib.otter_ref_ncnn_read, self.lib.otter_ref_last_error

    def net(self, otter_path, bin_path=None, use_packing=True):
        return RefNet(self, otter_path, bin_path, use_packing)

    def conv_layer(self, options, in_shape, wq, bias, weight_scales, in_scale, top_scale=1.0, use_packing=True):
        return RefConvLayer(self, options, in_shape, wq, bias, weight_scales, in_scale, top_scale, use_packing)


class RefConvLayer:
    """A real otter::ConvolutionLayer (options use the reference's own keys, Tensor/ConvolutionLayer.cpp:58-156)."""

    def __init__(self, ref, options, in_shape, wq, bias, weight_scales, in_scale, top_scale, use_packing):
        self.ref = ref
        opt = ";".join("%s=%s" % kv for kv in options.items()).encode()
        wq = np.ascontiguousarray(wq, np.int8)
        ws, b = _f32(np.atleast_1d(weight_scales)), _f32(bias)
        n, c, h, w = in_shape
        self.k = wq.shape[0]
        self.kh, self.kw = wq.shape[2], wq.shape[3]
        self.options = options
        self.h = ref.lib.otter_ref_conv_layer_create(opt, n, c, h, w, _p(wq, _i8p), _p(b, _f32p), _p(ws, _f32p),
                                                     C.c_int(ws.size), C.c_float(in_scale), C.c_float(top_scale),
                                                     C.c_int(int(use_packing)))
        if not self.h:
            raise RuntimeError("reference: " + ref.lib.otter_ref_last_error().decode(errors="replace"))
        self.int8_out = bool(ref.lib.otter_ref_conv_layer_int8_out(C.c_void_p(self.h)))

    def scale_in(self):
        out = np.empty(self.k, np.float32)
        self.ref.lib.otter_ref_conv_layer_scale_in(C.c_void_p(self.h), _p(out, _f32p))
        return out

    def forward(self, x, repeat=1, want_out=True):
        """Returns (out, seconds); seconds = min over `repeat` of the summed per-image forward time."""
        in_is_int8 = x.dtype == np.int8
        x = np.ascontiguousarray(x, np.int8 if in_is_int8 else np.float32)
        n, c, h, w = x.shape
        o = self.options
        g = lambda key, d: int(o.get(key, d))
        s, p, d = g("stride", 1), g("padding", 0), g("dilation", 1)
        oh = out_size(h, self.kh, g("stride_h", s), g("padding_h", p), g("dilation_h", d))
        ow = out_size(w, self.kw, g("stride_w", s), g("padding_w", p), g("dilation_w", d))
        out = np.empty((n, self.k, oh, ow), np.int8 if self.int8_out else np.float32) if want_out else None
        t = self.ref.lib.otter_ref_conv_layer_forward(C.c_void_p(self.h), x.ctypes.data_as(C.c_void_p),
                                                      C.c_int(int(in_is_int8)), n, h, w,
                                                      out.ctypes.data_as(C.c_void_p) if want_out else None,
                                                      C.c_int(repeat))
        if t < 0:
            raise RuntimeError("reference: " + self.ref.lib.otter_ref_last_error().decode(errors="replace"))
        return out, t

    def close(self):
        if self.h:
            self.ref.lib.otter_ref_conv_layer_destroy(C.c_void_p(self.h))
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class RefNet:
    """The reference's Net over a `.otter` description and an ncnn `.bin` (batch 1, every blob kept)."""

    def __init__(self, ref, otter_path, bin_path, use_packing):
        self.ref = ref
        L = ref.lib
        L.otter_ref_net_open.restype = C.c_void_p
        L.otter_ref_net_run.restype = C.c_double
        self.h = C.c_void_p(L.otter_ref_net_open(os.fsencode(otter_path), os.fsencode(bin_path) if bin_path else None,
                                                 C.c_int(int(use_packing))))
        if not self.h:
            raise RuntimeError("reference: " + L.otter_ref_last_error().decode(errors="replace"))

    def run(self, input_blob, x, names):
        """x: [1, C, H, W] fp32. Returns ({name: unpacked array}, seconds spent extracting names[0])."""
        x = _f32(x)
        assert x.ndim == 4 and x.shape[0] == 1
        L = self.ref.lib
        c_names = (C.c_char_p * len(names))(*[n.encode() for n in names])
        secs = L.otter_ref_net_run(self.h, input_blob.encode(), _p(x, _f32p), x.shape[1], x.shape[2], x.shape[3], c_names,
                                   len(names))
        if secs < 0:
            raise RuntimeError("reference: " + L.otter_ref_last_error().decode(errors="replace"))
        out = {}
        for i, n in enumerate(names):
            dims, is8 = (C.c_longlong * 4)(), C.c_int()
            self.ref._check(L.otter_ref_net_blob_info(self.h, i, dims, C.byref(is8)))
            a = np.empty(tuple(dims), np.int8 if is8.value else np.float32)
            self.ref._check(L.otter_ref_net_blob_copy(self.h, i, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes)))
            out[n] = a
        return out, secs

    def close(self):
        if self.h:
            self.ref.lib.otter_ref_net_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
