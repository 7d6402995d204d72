"""ctypes binding of the C facade over the C++ host layer (tensor_amd/host: Otter's Layer / ConvolutionLayer / Net
interface on the GPU). Used by the tests and the benchmark; a C++ program includes tensor_amd/host/otter_hip.hpp."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libotter_hip_host.so")

EXPORTS = ["otter_host_last_error", "otter_host_net_create", "otter_host_net_destroy", "otter_host_net_add_layer",
           "otter_host_net_compile", "otter_host_net_set_conv", "otter_host_net_get_scale_in",
           "otter_host_net_set_inner_product", "otter_host_net_run", "otter_host_session_create",
           "otter_host_session_pass", "otter_host_session_fetch", "otter_host_session_destroy",
           "otter_host_functional_chain", "otter_host_net_load_otter", "otter_host_net_load_weight",
           "otter_host_net_describe", "otter_host_net_conv_fp32_probe", "otter_host_net_eval", "otter_host_otter_dump", "otter_host_ncnn_read",
           "otter_host_chain_forward_count", "otter_host_block_forward_count"]


def load_cdll():
    if not os.path.exists(LIB_PATH):
        raise OSError("%s is not built: run tensor_amd/host/build.sh" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    lib.otter_host_last_error.restype = C.c_char_p
    lib.otter_host_net_create.restype = C.c_void_p
    lib.otter_host_session_create.restype = C.c_void_p
    lib.otter_host_session_fetch.restype = C.c_long
    lib.otter_host_net_describe.restype = C.c_long
    lib.otter_host_otter_dump.restype = C.c_long
    lib.otter_host_ncnn_read.restype = C.c_long
    lib.otter_host_chain_forward_count.restype = C.c_long
    lib.otter_host_block_forward_count.restype = C.c_long
    return lib


def block_forward_count():
    """Inverted-residual blocks the Nets of this process have run as one launch so far."""
    return load_cdll().otter_host_block_forward_count()


def chain_forward_count():
    """Runs of convolution layers that went through the C ABI's chain entry point as one launch, in this process."""
    return load_cdll().otter_host_chain_forward_count()


def _opts(d):
    return ";".join("%s=%s" % kv for kv in d.items()).encode()


class HostError(RuntimeError):
    pass


class Net:
    """otter::Net on the GPU. Layers are added with the reference's option dictionaries."""

    def __init__(self, use_packing_layout=True, lightmode=True):
        self.lib = load_cdll()
        self.h = C.c_void_p(self.lib.otter_host_net_create(int(use_packing_layout), int(lightmode)))
        if not self.h:
            raise HostError(self.lib.otter_host_last_error().decode())

    def _check(self, rc):
        if rc != 0:
            raise HostError(self.lib.otter_host_last_error().decode(errors="replace"))

    def add_layer(self, **options):
        self._check(self.lib.otter_host_net_add_layer(self.h, _opts(options)))

    def compile(self, initial=False):
        self._check(self.lib.otter_host_net_compile(self.h, int(initial)))

    def set_conv(self, name, wq, bias, weight_scales, in_scale, top_scale=1.0):
        wq = np.ascontiguousarray(wq, np.int8)
        ws = np.ascontiguousarray(np.atleast_1d(weight_scales), np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        f32p = C.POINTER(C.c_float)
        self._check(self.lib.otter_host_net_set_conv(
            self.h, name.encode(), wq.ctypes.data_as(C.c_void_p), b.ctypes.data_as(f32p) if b is not None else None,
            ws.ctypes.data_as(f32p), C.c_int(ws.size), C.c_float(in_scale), C.c_float(top_scale)))

    def conv_fp32_probe(self, name, on):
        """While on, an int8-output convolution runs as its fp32-output twin (calibration aid)."""
        self._check(self.lib.otter_host_net_conv_fp32_probe(self.h, name.encode(), int(on)))

    def scale_in(self, name, k):
        out = np.empty(k, np.float32)
        self._check(self.lib.otter_host_net_get_scale_in(self.h, name.encode(), out.ctypes.data_as(C.c_void_p)))
        return out

    def set_inner_product(self, name, weight, bias):
        w = np.ascontiguousarray(weight, np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        self._check(self.lib.otter_host_net_set_inner_product(
            self.h, name.encode(), w.ctypes.data_as(C.c_void_p), b.ctypes.data_as(C.c_void_p) if b is not None else None))

    def run(self, in_name, x, out_name, repeat=1):
        x = np.ascontiguousarray(x)
        n, c, h, w = x.shape
        cap = 1 << 28
        dtype, shape, secs = C.c_int(), (C.c_int64 * 4)(), C.c_double(0)
        buf = np.empty(cap // 16, np.uint8)
        # first ask for the shape only (out = NULL), then fetch
        self._check(self.lib.otter_host_net_run(self.h, in_name.encode(), x.ctypes.data_as(C.c_void_p),
                                                int(x.dtype == np.int8), n, c, h, w, out_name.encode(), None,
                                                C.c_size_t(0), C.byref(dtype), shape, 1, None))
        np_dt = [np.float32, np.int8, np.int32][dtype.value]
        out = np.empty(tuple(shape), np_dt)
        self._check(self.lib.otter_host_net_run(self.h, in_name.encode(), x.ctypes.data_as(C.c_void_p),
                                                int(x.dtype == np.int8), n, c, h, w, out_name.encode(),
                                                out.ctypes.data_as(C.c_void_p), C.c_size_t(out.nbytes), C.byref(dtype),
                                                shape, repeat, C.byref(secs)))
        del buf
        return (out, secs.value) if repeat > 1 else out

    def session(self, in_name, x, out_name):
        return Session(self, in_name, x, out_name)

    # ---- model files (Net::load_otter / Net::load_weight of the reference) ----
    def load_otter(self, path, initial=False):
        self._check(self.lib.otter_host_net_load_otter(self.h, os.fsencode(path), int(initial)))

    def load_weight(self, path, ncnn=True):
        self._check(self.lib.otter_host_net_load_weight(self.h, os.fsencode(path), int(ncnn)))

    def describe(self):
        """[(type, name, [bottom blobs], [top blobs], conv or None, top shape (N, C, H, W))], conv = dict(K, C, groups,
        kh, kw, bias_term, int8_scale_term)."""
        buf = C.create_string_buffer(1 << 22)
        n = self.lib.otter_host_net_describe(self.h, buf, C.c_size_t(len(buf)))
        if n < 0:
            raise HostError(self.lib.otter_host_last_error().decode())
        out = []
        for line in buf.value.decode().splitlines():
            f = line.split(" ")
            conv = None
            if len(f) > 8:
                conv = dict(zip(("K", "C", "groups", "kh", "kw", "bias_term", "int8_scale_term"), map(int, f[8:15])))
            out.append((f[0], f[1], [] if f[2] == "-" else f[2].split(","), [] if f[3] == "-" else f[3].split(","), conv,
                        tuple(map(int, f[4:8]))))
        return out

    def eval(self, inputs, out_name):
        """One pass with the blobs of `inputs` (name -> NCHW fp32 / int8 array) set beforehand; returns `out_name`
        unpacked (Extractor::input + Extractor::extract(name, type 0))."""
        names = [k.encode() for k in inputs]
        arrs = [np.ascontiguousarray(v) for v in inputs.values()]
        n = len(arrs)
        c_names = (C.c_char_p * n)(*names)
        c_ptrs = (C.c_void_p * n)(*[a.ctypes.data for a in arrs])
        c_i8 = (C.c_int * n)(*[int(a.dtype == np.int8) for a in arrs])
        c_shapes = (C.c_int64 * (4 * n))(*[d for a in arrs for d in a.shape])
        dtype, shape = C.c_int(), (C.c_int64 * 4)()
        cap = 1 << 28
        buf = np.empty(cap, np.uint8)
        self._check(self.lib.otter_host_net_eval(self.h, n, c_names, c_ptrs, c_i8, c_shapes, out_name.encode(),
                                                 buf.ctypes.data_as(C.c_void_p), C.c_size_t(cap), C.byref(dtype), shape))
        np_dt = [np.float32, np.int8, np.int32][dtype.value]
        count = int(np.prod(tuple(shape)))
        return buf[:count * np.dtype(np_dt).itemsize].view(np_dt).reshape(tuple(shape)).copy()

    def close(self):
        if self.h:
            self.lib.otter_host_net_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Session:
    def __init__(self, net, in_name, x, out_name):
        self.net = net
        x = np.ascontiguousarray(x)
        n, c, h, w = x.shape
        self.h = C.c_void_p(net.lib.otter_host_session_create(net.h, in_name.encode(), x.ctypes.data_as(C.c_void_p),
                                                              int(x.dtype == np.int8), n, c, h, w, out_name.encode()))
        if not self.h:
            raise HostError(net.lib.otter_host_last_error().decode())

    def run(self):
        self.net._check(self.net.lib.otter_host_session_pass(self.h))

    def fetch(self, shape, dtype):
        out = np.empty(shape, dtype)
        r = self.net.lib.otter_host_session_fetch(self.h, out.ctypes.data_as(C.c_void_p), C.c_size_t(out.nbytes))
        if r < 0:
            raise HostError(self.net.lib.otter_host_last_error().decode())
        return out

    def close(self):
        if self.h:
            self.net.lib.otter_host_session_destroy(self.h)
            self.h = None


def functional_chain(x, in_scale, wq, scale_in, bias, *, stride=1, pad=0, groups=1, int8_out=False, top_scale=1.0, act=0):
    """quantize_to_int8 -> convolution -> requantize | dequantize through the C++ functional API."""
    lib = load_cdll()
    x = np.ascontiguousarray(x, np.float32)
    wq = np.ascontiguousarray(wq, np.int8)
    n, c, h, w = x.shape
    k, _, kh, kw = wq.shape
    oh, ow = (h + 2 * pad - kh) // stride + 1, (w + 2 * pad - kw) // stride + 1
    acc = np.empty((n, k, oh, ow), np.int32)
    out = np.empty((n, k, oh, ow), np.int8 if int8_out else np.float32)
    si = np.ascontiguousarray(scale_in, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    rc = lib.otter_host_functional_chain(
        x.ctypes.data_as(C.c_void_p), n, c, h, w, C.c_float(in_scale), wq.ctypes.data_as(C.c_void_p), k, kh, kw, stride,
        pad, groups, si.ctypes.data_as(C.c_void_p), b.ctypes.data_as(C.c_void_p) if b is not None else None,
        int(int8_out), C.c_float(top_scale), act, acc.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    if rc != 0:
        raise HostError(lib.otter_host_last_error().decode(errors="replace"))
    return acc, out


def otter_dump(path, lib=None):
    """What the `.otter` parser makes of a file: 'N name', 'G key=value', 'T block', 'P key=value' lines."""
    lib = lib or load_cdll()
    buf = C.create_string_buffer(1 << 24)
    n = lib.otter_host_otter_dump(os.fsencode(path), buf, C.c_size_t(len(buf)))
    if n < 0:
        raise HostError(lib.otter_host_last_error().decode())
    return buf.raw[:n].decode(errors="surrogateescape")


def ncnn_read(path, shapes, kinds, reader=None, err=None):
    """Reads consecutive tensors from an ncnn `.bin` with InitializerNcnnFromDataReader. shapes: list of tuples
    (<= 4 dims), kinds: 0 weight (tagged) / 1 plain fp32. Returns ([array or None], bytes left in the file).
    `reader` / `err`: the same entry point of another library (the compiled reference's, in the tests)."""
    if reader is None:
        lib = load_cdll()
        reader, err = lib.otter_host_ncnn_read, lib.otter_host_last_error
    n = len(shapes)
    flat = (C.c_longlong * (4 * n))(*[(list(s) + [0] * 4)[:4][d] for s in shapes for d in range(4)])
    c_kinds = (C.c_int * n)(*kinds)
    dtypes = (C.c_int * n)()
    cap = 4 * sum(int(np.prod(s)) for s in shapes) + 64
    out = np.empty(cap, np.uint8)
    remain = C.c_longlong(-1)
    reader.restype = C.c_long
    used = reader(os.fsencode(path), n, flat, c_kinds, dtypes, out.ctypes.data_as(C.c_void_p), C.c_size_t(cap),
                  C.byref(remain))
    if used < 0:
        raise HostError(err().decode() if err else "ncnn_read failed")
    res, at = [], 0
    for s, dt in zip(shapes, dtypes):
        if dt < 0:
            res.append(None)
            continue
        np_dt = np.int8 if dt == 1 else np.float32
        nb = int(np.prod(s)) * np.dtype(np_dt).itemsize
        res.append(out[at:at + nb].view(np_dt).reshape(s).copy())
        at += nb
    return res, remain.value
