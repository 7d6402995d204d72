"""ctypes binding of include/otter_hip_int8.h. Fails loudly when the library or the GPU is missing:
there is no CPU fallback anywhere in this package."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libotter_hip_int8.so")

# otter_hip_layout
F32, F32_P4, F32_P8, I8, I8_P8, I32, I32_P4, I32_P8 = range(8)
OUT_I32, OUT_F32, OUT_I8 = 0, 1, 2
ROUND_SSE, ROUND_EXACT = 0, 1
ACT = {"": 0, None: 0, "Relu": 1, "LRelu": 2, "Relu6": 3, "Sigmoid": 4}

_PACK = {F32: 1, F32_P4: 4, F32_P8: 8, I8: 1, I8_P8: 8, I32: 1, I32_P4: 4, I32_P8: 8}
_NP = {F32: np.float32, F32_P4: np.float32, F32_P8: np.float32, I8: np.int8, I8_P8: np.int8, I32: np.int32,
       I32_P4: np.int32, I32_P8: np.int32}


def layout_pack(layout):
    return _PACK[layout]


def layout_dtype(layout):
    return _NP[layout]


def layout_for(dtype, pack):
    base = {np.dtype(np.float32): F32, np.dtype(np.int8): I8, np.dtype(np.int32): I32}[np.dtype(dtype)]
    return base + {1: 0, 4: 1, 8: 2 if base != I8 else 1}[pack]


def pack_np(a, p):
    """[N,C,H,W] -> the reference's packed storage [N,C/p,H,W,p] (numpy, host side test helper)."""
    if p == 1:
        return np.ascontiguousarray(a)
    n, c, h, w = a.shape
    return np.ascontiguousarray(a.reshape(n, c // p, p, h, w).transpose(0, 1, 3, 4, 2))


def unpack_np(a, p, shape):
    if p == 1:
        return np.ascontiguousarray(a).reshape(shape)
    n, c, h, w = shape
    return np.ascontiguousarray(a.reshape(n, c // p, h, w, p).transpose(0, 1, 4, 2, 3)).reshape(shape)


class ConvDesc(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("in_channels", "out_channels", "kernel_h", "kernel_w", "stride_h", "stride_w",
                                       "pad_h", "pad_w", "dilation_h", "dilation_w", "groups", "activation_type")] + \
               [("activation_param0", C.c_float), ("out_kind", C.c_int), ("out_round_mode", C.c_int),
                ("in_round_mode", C.c_int)]


class HipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("otter_hip error %d: %s" % (code, msg))
        self.code = code


EXPORTS = ["otter_hip_init", "otter_hip_shutdown", "otter_hip_last_error", "otter_hip_device_info",
           "otter_hip_shader_clock_mhz", "otter_hip_malloc",
           "otter_hip_free", "otter_hip_memcpy_h2d", "otter_hip_memcpy_d2h", "otter_hip_stream_create",
           "otter_hip_stream_destroy", "otter_hip_stream_synchronize", "otter_hip_conv_create",
           "otter_hip_conv_destroy", "otter_hip_conv_output_shape", "otter_hip_conv_default_out_layout",
           "otter_hip_conv_workspace_bytes", "otter_hip_conv_forward", "otter_hip_conv_kernel_kind",
           "otter_hip_quantize", "otter_hip_dequantize", "otter_hip_requantize", "otter_hip_repack",
           "otter_hip_conv_set_tile", "otter_hip_eltwise_add", "otter_hip_activation", "otter_hip_global_avgpool",
           "otter_hip_inner_product", "otter_hip_eltwise_add_quantize", "otter_hip_copy_channels",
           "otter_hip_channel_shuffle", "otter_hip_maxpool2d", "otter_hip_upsample2d", "otter_hip_shuffle2_split",
           "otter_hip_conv_forward_twin", "otter_hip_conv_forward_residual",
           "otter_hip_copy_channels_quantize", "otter_hip_channel_shuffle_quantize",
           "otter_hip_concat_channels", "otter_hip_conv_forward_static", "otter_hip_conv3x3_halo_plan", "otter_hip_conv_chain_workspace_bytes",
           "otter_hip_conv_chain_forward", "otter_hip_conv_chain_status", "otter_hip_conv_chain_launches",
           "otter_hip_conv_chain_last_launches", "otter_hip_conv_chain_clock_mhz",
           "otter_hip_conv_chain_set_min_tiles", "otter_hip_conv_block_launches", "otter_hip_conv_block_workspace_bytes",
           "otter_hip_conv_block_forward", "otter_hip_conv_block_set_plan", "otter_hip_conv_block_set_always", "otter_hip_conv_block_set_pair",
           "otter_hip_conv_avgpool_launches", "otter_hip_conv_avgpool_workspace_bytes", "otter_hip_conv_forward_avgpool",
           "otter_hip_conv_block_plan"]


def load_cdll():
    if not os.path.exists(LIB_PATH):
        raise OSError("%s is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
                      "(tensor_amd/csrc/build.sh)" % LIB_PATH)
    return C.CDLL(LIB_PATH)


class Library:
    """The GPU library on cuda:0. Tensors are torch CUDA tensors holding the reference's packed storage."""

    def __init__(self, device=0):
        import torch
        self.torch = torch
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the int8 convolution path has no CPU fallback")
        L = self.lib = load_cdll()
        L.otter_hip_last_error.restype = C.c_char_p
        L.otter_hip_conv_workspace_bytes.restype = C.c_size_t
        L.otter_hip_conv_chain_workspace_bytes.restype = C.c_size_t
        L.otter_hip_conv_block_workspace_bytes.restype = C.c_size_t
        L.otter_hip_conv_avgpool_workspace_bytes.restype = C.c_size_t
        self.device = torch.device("cuda", device)
        self._check(L.otter_hip_init(C.c_int(device)))

    # -- plumbing -------------------------------------------------------------------------------------
    def _check(self, rc):
        if rc != 0:
            raise HipError(rc, self.lib.otter_hip_last_error().decode(errors="replace"))

    def stream(self):
        return C.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def to_device(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).to(self.device)

    def empty(self, count, dtype):
        t = {np.float32: self.torch.float32, np.int8: self.torch.int8, np.int32: self.torch.int32}[dtype]
        return self.torch.empty(int(count), dtype=t, device=self.device)

    @staticmethod
    def ptr(t):
        return C.c_void_p(t.data_ptr())

    def device_info(self):
        v = [C.c_int() for _ in range(4)]
        self._check(self.lib.otter_hip_device_info(*[C.byref(x) for x in v]))
        return dict(compute_units=v[0].value, clock_mhz=v[1].value, mem_clock_mhz=v[2].value, mem_bus_bits=v[3].value)

    def shader_clock_mhz(self):
        """otter_hip_shader_clock_mhz: the shader clock under int8 matrix load, measured now on the current stream."""
        v = C.c_float(0)
        self._check(self.lib.otter_hip_shader_clock_mhz(self.stream(), C.byref(v)))
        return float(v.value)

    # -- standalone ops (device tensors in packed storage) ------------------------------------------------
    def quantize(self, src, src_layout, shape, scales, round_mode, dst_layout, dst=None):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, np.int8) if dst is None else dst
        self._check(self.lib.otter_hip_quantize(self.ptr(src), src_layout, n, c, h, w, self.ptr(scales),
                                                C.c_int(scales.numel()), round_mode, self.ptr(dst), dst_layout,
                                                self.stream()))
        return dst

    def dequantize(self, src, src_layout, shape, scale, bias, dst_layout, dst=None):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, np.float32) if dst is None else dst
        self._check(self.lib.otter_hip_dequantize(self.ptr(src), src_layout, n, c, h, w, self.ptr(scale),
                                                  C.c_int(scale.numel()), self.ptr(bias) if bias is not None else None,
                                                  C.c_int(0 if bias is None else bias.numel()), self.ptr(dst),
                                                  dst_layout, self.stream()))
        return dst

    def requantize(self, src, src_layout, shape, scale_in, scale_out, bias, act, act_p0, round_mode, dst_layout,
                   dst=None):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, np.int8) if dst is None else dst
        self._check(self.lib.otter_hip_requantize(
            self.ptr(src), src_layout, n, c, h, w, self.ptr(scale_in), C.c_int(scale_in.numel()), self.ptr(scale_out),
            C.c_int(scale_out.numel()), self.ptr(bias) if bias is not None else None,
            C.c_int(0 if bias is None else bias.numel()), C.c_int(act), C.c_float(act_p0), C.c_int(round_mode),
            self.ptr(dst), dst_layout, self.stream()))
        return dst

    def repack(self, src, src_layout, shape, dst_layout, dst=None):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, layout_dtype(src_layout)) if dst is None else dst
        self._check(self.lib.otter_hip_repack(self.ptr(src), src_layout, n, c, h, w, self.ptr(dst), dst_layout,
                                              self.stream()))
        return dst

    # -- fp32 layout glue (device tensors in packed storage; every op takes any fp32 layout on either side) ------
    def copy_channels(self, src, src_layout, src_c, src_c0, dst, dst_layout, dst_c, dst_c0, count, n, h, w):
        self._check(self.lib.otter_hip_copy_channels(self.ptr(src), src_layout, src_c, src_c0, self.ptr(dst), dst_layout,
                                                     dst_c, dst_c0, count, n, h, w, self.stream()))
        return dst

    def copy_channels_quantize(self, src, src_layout, src_c, src_c0, dst, dst_layout, dst_c, dst_c0, count, n, h, w, dst_q,
                               scale, round_mode):
        self._check(self.lib.otter_hip_copy_channels_quantize(
            self.ptr(src), src_layout, src_c, src_c0, self.ptr(dst), dst_layout, dst_c, dst_c0, count, n, h, w,
            self.ptr(dst_q), C.c_float(scale), round_mode, self.stream()))
        return dst, dst_q

    def concat_channels(self, srcs, src_layouts, src_channels, n, h, w, dst_layout, scale=None, round_mode=ROUND_SSE):
        """Concat over channels in one launch; with scale also the Byte8 quantization of the result."""
        k = len(srcs)
        total = sum(src_channels)
        dst = self.empty(n * total * h * w, np.float32)
        q = self.empty(n * total * h * w, np.int8) if scale is not None else None
        ptrs = (C.c_void_p * k)(*[t.data_ptr() for t in srcs])
        self._check(self.lib.otter_hip_concat_channels(ptrs, (C.c_int * k)(*src_layouts), (C.c_int * k)(*src_channels), k,
                                                       self.ptr(dst), dst_layout, n, h, w,
                                                       self.ptr(q) if q is not None else None, C.c_float(scale or 0.0),
                                                       round_mode, self.stream()))
        return dst, q

    def channel_shuffle(self, src, src_layout, shape, groups, dst_layout):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, np.float32)
        self._check(self.lib.otter_hip_channel_shuffle(self.ptr(src), src_layout, self.ptr(dst), dst_layout, n, c, h, w,
                                                       groups, self.stream()))
        return dst

    def channel_shuffle_quantize(self, src, shape, groups, scale, round_mode, layout=F32_P8):
        n, c, h, w = shape
        dst = self.empty(n * c * h * w, np.float32)
        q = self.empty(n * c * h * w, np.int8)
        self._check(self.lib.otter_hip_channel_shuffle_quantize(self.ptr(src), layout, self.ptr(dst), layout, n, c, h, w,
                                                                groups, self.ptr(q), C.c_float(scale), round_mode,
                                                                self.stream()))
        return dst, q

    def shuffle2_split(self, a, b, n, channels_each, h, w, scale=None, round_mode=0, a_layout=F32_P8, b_layout=F32_P8):
        c1 = self.empty(n * channels_each * h * w, np.float32)
        c2 = self.empty(n * channels_each * h * w, np.float32)
        q2 = self.empty(n * channels_each * h * w, np.int8) if scale is not None else None
        self._check(self.lib.otter_hip_shuffle2_split(self.ptr(a), a_layout, self.ptr(b), b_layout, n, channels_each, h, w, self.ptr(c1),
                                                      self.ptr(c2), self.ptr(q2) if q2 is not None else None,
                                                      C.c_float(scale or 0.0), round_mode, self.stream()))
        return (c1, c2, q2) if scale is not None else (c1, c2)

    def maxpool2d(self, src, src_layout, shape, kernel, stride, pad, dil, out_hw, pad_value, dst_layout):
        n, c, h, w = shape
        dst = self.empty(n * c * out_hw[0] * out_hw[1], np.float32)
        self._check(self.lib.otter_hip_maxpool2d(self.ptr(src), src_layout, n, c, h, w, kernel[0], kernel[1], stride[0],
                                                 stride[1], pad[0], pad[1], dil[0], dil[1], out_hw[0], out_hw[1],
                                                 C.c_float(pad_value), self.ptr(dst), dst_layout, self.stream()))
        return dst

    def upsample2d(self, src, src_layout, shape, out_hw, mode, align_corner, dst_layout):
        n, c, h, w = shape
        dst = self.empty(n * c * out_hw[0] * out_hw[1], np.float32)
        self._check(self.lib.otter_hip_upsample2d(self.ptr(src), src_layout, n, c, h, w, out_hw[0], out_hw[1], mode,
                                                  int(align_corner), self.ptr(dst), dst_layout, self.stream()))
        return dst

    def inner_product(self, x, n, in_features, weight, bias, out_features):
        """otter_hip_inner_product: y[n][o] = sum_i x[n][i] * weight[o][i] + bias[o] (device tensors; bias may be None)."""
        y = self.empty(n * out_features, np.float32)
        self._check(self.lib.otter_hip_inner_product(self.ptr(x), n, in_features, self.ptr(weight),
                                                     self.ptr(bias) if bias is not None else None, out_features,
                                                     self.ptr(y), self.stream()))
        return y

    def eltwise_add_quantize(self, a, b, layout, shape, scale, round_mode):
        n, c, h, w = shape
        out = self.empty(n * c * h * w, np.float32)
        q = self.empty(n * c * h * w, np.int8)
        self._check(self.lib.otter_hip_eltwise_add_quantize(self.ptr(a), self.ptr(b), layout, n, c, h, w, C.c_float(scale),
                                                            round_mode, self.ptr(out), self.ptr(q), self.stream()))
        return out, q

    def conv(self, **kw):
        return Conv(self, **kw)

    def global_avgpool(self, x, layout, n, c, h, w):
        """otter_hip_global_avgpool: the mean over H*W of an fp32 blob, [n, c]."""
        out = self.empty(n * c, np.float32)
        self._check(self.lib.otter_hip_global_avgpool(self.ptr(x), layout, n, c, h, w, self.ptr(out), self.stream()))
        return out

    def conv_chain(self, convs, x, n, h, w, out=None, workspace=None):
        """otter_hip_conv_chain_forward: x (int8 Byte8) through the layers `convs`, intermediate blobs in `workspace`."""
        hs = (C.c_void_p * len(convs))(*[c.h for c in convs])
        ws_bytes = self.lib.otter_hip_conv_chain_workspace_bytes(hs, len(convs), n, h, w)
        if ws_bytes and workspace is None:
            workspace = self.empty(ws_bytes, np.int8)
        oh, ow = h, w
        for c in convs:
            oh, ow = c.out_hw(oh, ow)
        if out is None:
            out = self.empty(n * convs[-1].K * oh * ow, np.int8)
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0  # what the buffer really holds
        self._check(self.lib.otter_hip_conv_chain_forward(hs, len(convs), self.ptr(x), n, h, w, self.ptr(out),
                                                          self.ptr(workspace) if workspace is not None else None,
                                                          C.c_size_t(ws_bytes), self.stream()))
        return out

    def conv_block(self, expand, dw, project, x, n, h, w, residual=None, q_scale=None, q_round_mode=ROUND_SSE, out=None,
                   q=None, workspace=None):
        """otter_hip_conv_block_forward: x (int8 Byte8) through expand -> depthwise -> project (+ residual), and with
        q_scale the Byte8 quantization of the result. Returns (out, q or None)."""
        oh, ow = dw.out_hw(*expand.out_hw(h, w))
        oh, ow = project.out_hw(oh, ow)
        f32 = project.out_kind == OUT_F32
        out_layout = F32_P4 if f32 else I8_P8
        if out is None:
            out = self.empty(n * project.K * oh * ow, np.float32 if f32 else np.int8)
        if q is None and q_scale is not None:
            q = self.empty(n * project.K * oh * ow, np.int8)
        ws_bytes = self.lib.otter_hip_conv_block_workspace_bytes(expand.h, dw.h, project.h, n, h, w)
        if ws_bytes and workspace is None:
            workspace = self.empty(ws_bytes, np.int8)
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0  # what the buffer really holds
        self._check(self.lib.otter_hip_conv_block_forward(
            expand.h, dw.h, project.h, self.ptr(x), n, h, w, self.ptr(residual) if residual is not None else None,
            self.ptr(out), out_layout, self.ptr(q) if q is not None else None, C.c_float(q_scale or 0.0), q_round_mode,
            self.ptr(workspace) if workspace is not None else None, C.c_size_t(ws_bytes), self.stream()))
        return out, q

    def conv_block_set_always(self, on):
        """otter_hip_conv_block_set_always: returns the previous setting."""
        return self.lib.otter_hip_conv_block_set_always(int(on))

    def conv_block_set_pair(self, mode):
        """otter_hip_conv_block_set_pair: returns the previous setting."""
        return self.lib.otter_hip_conv_block_set_pair(int(mode))

    def conv_block_launches(self, expand, dw, project, n, h, w):
        r = self.lib.otter_hip_conv_block_launches(expand.h, dw.h, project.h, n, h, w)
        self._check(min(r, 0))
        return r

    def conv_chain_launches(self, convs, n, h, w):
        hs = (C.c_void_p * len(convs))(*[c.h for c in convs])
        r = self.lib.otter_hip_conv_chain_launches(hs, len(convs), n, h, w)
        self._check(min(r, 0))
        return r

    def conv_chain_set_min_tiles(self, tiles):
        """otter_hip_conv_chain_set_min_tiles: returns the previous threshold."""
        return self.lib.otter_hip_conv_chain_set_min_tiles(int(tiles))

    def conv_chain_last_launches(self):
        """otter_hip_conv_chain_last_launches: the launches the last chain call of this thread actually made."""
        return self.lib.otter_hip_conv_chain_last_launches()

    def conv_chain_clock_mhz(self):
        """otter_hip_conv_chain_clock_mhz: the shader clock of the last single-launch chain (synchronizes); 0 if none."""
        v = C.c_float(0)
        self._check(self.lib.otter_hip_conv_chain_clock_mhz(C.byref(v)))
        return float(v.value)

    def conv_chain_gave_up(self):
        """otter_hip_conv_chain_status: synchronizes; True if a chain launch since the last call gave up a wait."""
        v = C.c_int(0)
        self._check(self.lib.otter_hip_conv_chain_status(C.byref(v)))
        return bool(v.value)


class Conv:
    """otter_hip_conv_t. Arguments follow otter::ConvolutionLayer's members (Tensor/ConvolutionLayer.hpp:40-77)."""

    def __init__(self, lib, *, wq, scale_in, bias=None, in_scale=1.0, out_scale=None, stride=(1, 1), pad=(0, 0),
                 dil=(1, 1), groups=1, act=0, act_p0=0.0, out_kind=OUT_I32, out_round=ROUND_SSE, in_round=ROUND_SSE):
        self.L = lib
        wq = np.ascontiguousarray(wq, np.int8)
        k, cg, kh, kw = wq.shape
        self.K, self.C, self.kh, self.kw = k, cg * groups, kh, kw
        self.stride, self.pad, self.dil, self.groups, self.out_kind = stride, pad, dil, groups, out_kind
        d = ConvDesc(cg * groups, k, kh, kw, stride[0], stride[1], pad[0], pad[1], dil[0], dil[1], groups, act,
                     act_p0, out_kind, out_round, in_round)
        si = np.ascontiguousarray(scale_in, np.float32)
        assert si.size == k
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        so = None if out_scale is None else np.ascontiguousarray(np.atleast_1d(out_scale), np.float32)
        self.h = C.c_void_p()
        f32p = C.POINTER(C.c_float)
        lib._check(lib.lib.otter_hip_conv_create(
            C.byref(d), wq.ctypes.data_as(C.c_void_p), si.ctypes.data_as(f32p),
            b.ctypes.data_as(f32p) if b is not None else None, C.c_float(in_scale),
            so.ctypes.data_as(f32p) if so is not None else None, C.c_int(0 if so is None else so.size),
            C.byref(self.h)))

    def out_hw(self, h, w):
        oh, ow = C.c_int(), C.c_int()
        self.L._check(self.L.lib.otter_hip_conv_output_shape(self.h, h, w, C.byref(oh), C.byref(ow)))
        return oh.value, ow.value

    def default_out_layout(self):
        return self.L.lib.otter_hip_conv_default_out_layout(self.h)

    def kernel_kind(self, in_layout, n, h, w, out_layout):
        return self.L.lib.otter_hip_conv_kernel_kind(self.h, in_layout, n, h, w, out_layout)

    def set_tile(self, tm, tn):
        self.L._check(self.L.lib.otter_hip_conv_set_tile(self.h, tm, tn))

    def set_block_plan(self, rows_per_band, slice_channels, split=0):
        self.L._check(self.L.lib.otter_hip_conv_block_set_plan(self.h, rows_per_band, slice_channels, split))

    def forward(self, x, in_layout, n, h, w, out_layout=None, out=None, workspace=None):
        out_layout = self.default_out_layout() if out_layout is None else out_layout
        oh, ow = self.out_hw(h, w)
        if out is None:
            out = self.L.empty(n * self.K * oh * ow, layout_dtype(out_layout))
        ws_bytes = self.L.lib.otter_hip_conv_workspace_bytes(self.h, in_layout, n, h, w)
        if ws_bytes and workspace is None:
            workspace = self.L.empty(ws_bytes, np.int8)
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0  # what the buffer really holds
        self.L._check(self.L.lib.otter_hip_conv_forward(
            self.h, self.L.ptr(x), in_layout, n, h, w, self.L.ptr(out), out_layout,
            self.L.ptr(workspace) if workspace is not None else None, C.c_size_t(ws_bytes), self.L.stream()))
        return out

    def avgpool_launches(self, in_layout, n, h, w):
        r = self.L.lib.otter_hip_conv_avgpool_launches(self.h, in_layout, n, h, w)
        self.L._check(min(r, 0))
        return r

    def forward_avgpool(self, x, in_layout, n, h, w):
        """otter_hip_conv_forward_avgpool: the layer's fp32 result averaged over the image, [n, K]."""
        out = self.L.empty(n * self.K, np.float32)
        ws_bytes = self.L.lib.otter_hip_conv_avgpool_workspace_bytes(self.h, in_layout, n, h, w)
        workspace = self.L.empty(ws_bytes, np.int8) if ws_bytes else None
        self.L._check(self.L.lib.otter_hip_conv_forward_avgpool(
            self.h, self.L.ptr(x), in_layout, n, h, w, self.L.ptr(out),
            self.L.ptr(workspace) if workspace is not None else None, C.c_size_t(ws_bytes), self.L.stream()))
        return out

    def forward_static(self, x, in_layout, n, h, w, out_layout=None, out=None):
        """otter_hip_conv_forward_static: the workspace is the library's static device array (no allocation inside)."""
        out_layout = self.default_out_layout() if out_layout is None else out_layout
        oh, ow = self.out_hw(h, w)
        if out is None:
            out = self.L.empty(n * self.K * oh * ow, layout_dtype(out_layout))
        self.L._check(self.L.lib.otter_hip_conv_forward_static(
            self.h, self.L.ptr(x), in_layout, n, h, w, self.L.ptr(out), out_layout, self.L.stream()))
        return out

    def forward_twin(self, x, in_layout, n, h, w, q_scale, q_round_mode, out_layout=None):
        """fp32 result and its Byte8 quantization for the int8 convolutions that read it (otter_hip_conv_forward_twin)"""
        out_layout = self.default_out_layout() if out_layout is None else out_layout
        oh, ow = self.out_hw(h, w)
        out = self.L.empty(n * self.K * oh * ow, layout_dtype(out_layout))
        q = self.L.empty(n * self.K * oh * ow, np.int8)
        ws_bytes = self.L.lib.otter_hip_conv_workspace_bytes(self.h, in_layout, n, h, w)
        workspace = self.L.empty(ws_bytes, np.int8) if ws_bytes else None
        self.L._check(self.L.lib.otter_hip_conv_forward_twin(
            self.h, self.L.ptr(x), in_layout, n, h, w, self.L.ptr(out), out_layout, self.L.ptr(q), C.c_float(q_scale),
            q_round_mode, self.L.ptr(workspace) if workspace is not None else None, C.c_size_t(ws_bytes),
            self.L.stream()))
        return out, q

    def forward_residual(self, x, in_layout, n, h, w, residual, q_scale=None, q_round_mode=ROUND_SSE, out_layout=None):
        """activation(convolution) + residual, and with q_scale the Byte8 quantization of that sum
        (otter_hip_conv_forward_residual). Returns (sum, q or None)."""
        out_layout = self.default_out_layout() if out_layout is None else out_layout
        oh, ow = self.out_hw(h, w)
        out = self.L.empty(n * self.K * oh * ow, layout_dtype(out_layout))
        q = self.L.empty(n * self.K * oh * ow, np.int8) if q_scale is not None else None
        ws_bytes = self.L.lib.otter_hip_conv_workspace_bytes(self.h, in_layout, n, h, w)
        workspace = self.L.empty(ws_bytes, np.int8) if ws_bytes else None
        self.L._check(self.L.lib.otter_hip_conv_forward_residual(
            self.h, self.L.ptr(x), in_layout, n, h, w, self.L.ptr(residual), self.L.ptr(out), out_layout,
            self.L.ptr(q) if q is not None else None, C.c_float(q_scale or 0.0), q_round_mode,
            self.L.ptr(workspace) if workspace is not None else None, C.c_size_t(ws_bytes), self.L.stream()))
        return out, q

    def close(self):
        if self.h:
            self.L.lib.otter_hip_conv_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
