// Scalar direct int8 convolution: the catch-all for shapes the MFMA / depthwise kernels do not take
// (C % 8 != 0 with an unpacked blob, grouped non-depthwise convolutions, K not a multiple of the vector
// width of the requested output layout). One thread per output element, any input / output layout.
// States the same arithmetic as the reference's own scalar kernel (Tensor/ConvolutionMM2D.cpp:553-649).
#include "common.hpp"

namespace ohip {

__global__ void __launch_bounds__(256) conv_direct_kernel(const int8_t* __restrict__ x, int in_pack,
                                                          const int8_t* __restrict__ wt, void* __restrict__ out,
                                                          ConvGeom g, Epilogue ep) {
    const int OHW = g.OH * g.OW;
    const size_t total = (size_t)g.N * g.K * OHW;
    const int cg = g.C / g.groups, kg = g.K / g.groups;
    const int out_pack = layout_pack(ep.out_layout);
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int pix = (int)(idx % OHW);
        const size_t r = idx / OHW;
        const int k = (int)(r % g.K);
        const int n = (int)(r / g.K);
        const int oy = pix / g.OW, ox = pix % g.OW;
        const int grp = k / kg;
        int acc = 0;
        for (int q = 0; q < cg; ++q) {
            const int c = grp * cg + q;
            const int8_t* wp = wt + ((size_t)k * cg + q) * g.kh * g.kw;
            for (int u = 0; u < g.kh; ++u) {
                const int iy = oy * g.sh - g.ph + u * g.dh;
                if (iy < 0 || iy >= g.H) continue;
                for (int v = 0; v < g.kw; ++v) {
                    const int ix = ox * g.sw - g.pw + v * g.dw;
                    if (ix < 0 || ix >= g.W) continue;
                    acc += (int)x[elem_offset(in_pack, n, c, iy * g.W + ix, g.C, g.H * g.W)] * (int)wp[u * g.kw + v];
                }
            }
        }
        const size_t o = elem_offset(out_pack, n, k, pix, g.K, OHW);
        if (ep.out_kind == OTTER_HIP_OUT_I32) {
            ((int32_t*)out)[o] = acc;
        } else if (ep.out_kind == OTTER_HIP_OUT_F32) {
            float v = dequant_rt(acc, ep.scale_in[k], ep.bias ? ep.bias[k] : 0.f, ep.bias != nullptr);
            ((float*)out)[o] = activate(v, ep.act, ep.act_p0);
        } else {
            ((int8_t*)out)[o] = (int8_t)requant_rt(acc, ep.scale_in[k], ep.bias ? ep.bias[k] : 0.f, ep.bias != nullptr,
                                                   ep.act, ep.act_p0, ep.scale_out[k], ep.round_mode);
        }
    }
}

hipError_t run_conv_direct(const int8_t* x, int in_pack, const int8_t* wt, void* out, const ConvGeom& g,
                           const Epilogue& ep, hipStream_t stream) {
    const size_t total = (size_t)g.N * g.K * g.OH * g.OW;
    if (total == 0) return hipSuccess;
    size_t blocks = (total + 255) / 256;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    hipLaunchKernelGGL(conv_direct_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, in_pack, wt, out, g, ep);
    return hipGetLastError();
}

}  // namespace ohip
