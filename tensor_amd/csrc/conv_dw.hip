// Depthwise int8 convolution on the reference's Byte8 layout: a bandwidth-bound kernel, no MFMA.
//
// One (image, channel octet) plane [H, W, 8 bytes] is independent of every other, so a workgroup works inside
// one plane: its 8 x maxk weights and its 8 scale/bias values are wave-uniform and live in scalar registers.
// A lane owns one output column and walks down a strip of output rows, so consecutive lanes read consecutive
// 8-byte pixels (a wave reads 512 contiguous bytes per tap column) and every input row is fetched once per
// strip and reused from registers for the rows below it.
// The multiply-accumulate uses v_dot4_i32_i8 against a weight word that holds the tap weight in the byte of
// its channel and zeros elsewhere: one instruction per (tap, channel) with no byte unpacking of the input.
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v2i __attribute__((ext_vector_type(2)));

// weight [C, 1, kh, kw] int8 -> [C/8][maxk][8] int32, entry = (w & 0xff) << (8 * (c % 4))
size_t dw_packed_weight_bytes(int C, int kh, int kw) { return (size_t)(C / 8) * kh * kw * 8 * sizeof(int32_t); }

void dw_pack_weights(const int8_t* w, int C, int kh, int kw, int32_t* dst) {
    const int maxk = kh * kw;
    for (int o = 0; o < C / 8; ++o)
        for (int t = 0; t < maxk; ++t)
            for (int e = 0; e < 8; ++e) {
                const uint32_t b = (uint8_t)w[(size_t)(o * 8 + e) * maxk + t];
                dst[((size_t)o * maxk + t) * 8 + e] = (int32_t)(b << (8 * (e % 4)));
            }
}

__device__ __forceinline__ void mac8(int (&acc)[8], v2i px, const int* __restrict__ wm) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = __builtin_amdgcn_sdot4(px[0], wm[e], acc[e], false);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[4 + e] = __builtin_amdgcn_sdot4(px[1], wm[4 + e], acc[4 + e], false);
}

// 3x3, dilation 1, stride S (1 or 2): R output rows per lane with the input rows kept in registers.
template <int S, int R>
__global__ void __launch_bounds__(256) conv_dw3x3_kernel(const int8_t* __restrict__ x, const int32_t* __restrict__ wmask,
                                                         void* __restrict__ out, ConvGeom g, Epilogue ep, int n_strips) {
    const int C8 = g.C / 8;
    const int plane = blockIdx.y;
    const int n = plane / C8, o = plane % C8;
    const int t = blockIdx.x * 256 + threadIdx.x;
    const int ox = t % g.OW;
    const int strip = t / g.OW;
    if (strip >= n_strips) return;

    int wm[72];
    const int* wsrc = wmask + (size_t)o * 72;
#pragma unroll
    for (int i = 0; i < 72; ++i) wm[i] = wsrc[i];
    float si[8], bi[8], so[8];
    const bool has_bias = ep.bias != nullptr;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        si[e] = ep.scale_in[o * 8 + e];
        bi[e] = has_bias ? ep.bias[o * 8 + e] : 0.f;
        so[e] = ep.scale_out ? ep.scale_out[o * 8 + e] : 1.f;
    }

    const int8_t* xp = x + (size_t)plane * g.H * g.W * 8;
    const int ix0 = ox * S - g.pw;
    const bool cok[3] = {ix0 >= 0 && ix0 < g.W, ix0 + 1 >= 0 && ix0 + 1 < g.W, ix0 + 2 >= 0 && ix0 + 2 < g.W};
    const int oy0 = strip * R;
    const int OHW = g.OH * g.OW;

    auto load_row = [&](int iy, v2i (&row)[3]) {
        const bool rok = iy >= 0 && iy < g.H;
        const int8_t* rp = xp + ((size_t)iy * g.W + ix0) * 8;
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            v2i v = {0, 0};
            if (rok && cok[c]) v = *reinterpret_cast<const v2i*>(rp + c * 8);
            row[c] = v;
        }
    };

    constexpr int NROWS = (R - 1) * S + 3;  // input rows a strip touches
    v2i rows[NROWS][3];
    const int iy_base = oy0 * S - g.ph;
#pragma unroll
    for (int r = 0; r < NROWS; ++r) load_row(iy_base + r, rows[r]);  // rows outside the image read as zero
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int oy = oy0 + r;
        if (oy >= g.OH) break;
        int acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 3; ++u)
#pragma unroll
            for (int v = 0; v < 3; ++v) mac8(acc, rows[r * S + u][v], &wm[(u * 3 + v) * 8]);
        epilogue_store8(out, ep, n, o * 8, oy * g.OW + ox, g.K, OHW, acc, si, bi, so);
    }
}

// any kernel size / stride / dilation: one output pixel per lane
__global__ void __launch_bounds__(256) conv_dw_generic_kernel(const int8_t* __restrict__ x,
                                                              const int32_t* __restrict__ wmask, void* __restrict__ out,
                                                              ConvGeom g, Epilogue ep) {
    const int C8 = g.C / 8;
    const int plane = blockIdx.y;
    const int n = plane / C8, o = plane % C8;
    const int OHW = g.OH * g.OW;
    const int pix = blockIdx.x * 256 + threadIdx.x;
    if (pix >= OHW) return;
    const int oy = pix / g.OW, ox = pix % g.OW;
    const int maxk = g.kh * g.kw;
    const int* wsrc = wmask + (size_t)o * maxk * 8;
    const int8_t* xp = x + (size_t)plane * g.H * g.W * 8;
    int acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int u = 0; u < g.kh; ++u) {
        const int iy = oy * g.sh - g.ph + u * g.dh;
        if (iy < 0 || iy >= g.H) continue;
        for (int v = 0; v < g.kw; ++v) {
            const int ix = ox * g.sw - g.pw + v * g.dw;
            if (ix < 0 || ix >= g.W) continue;
            const v2i px = *reinterpret_cast<const v2i*>(xp + ((size_t)iy * g.W + ix) * 8);
            mac8(acc, px, wsrc + (u * g.kw + v) * 8);
        }
    }
    float si[8], bi[8], so[8];
    const bool has_bias = ep.bias != nullptr;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        si[e] = ep.scale_in[o * 8 + e];
        bi[e] = has_bias ? ep.bias[o * 8 + e] : 0.f;
        so[e] = ep.scale_out ? ep.scale_out[o * 8 + e] : 1.f;
    }
    epilogue_store8(out, ep, n, o * 8, pix, g.K, OHW, acc, si, bi, so);
}

hipError_t run_conv_dw(const int8_t* x, const int32_t* wmask, void* out, const ConvGeom& g, const Epilogue& ep,
                       hipStream_t stream) {
    const int planes = g.N * (g.C / 8);
    if (planes == 0 || g.OH * g.OW == 0) return hipSuccess;
    if (planes > 65535) return hipErrorInvalidValue;  // grid.y limit; the caller splits the batch
    const bool k3 = g.kh == 3 && g.kw == 3 && g.dh == 1 && g.dw == 1 && g.sh == g.sw && (g.sh == 1 || g.sh == 2);
    if (k3) {
        constexpr int R1 = 8, R2 = 4;
        const int R = g.sh == 1 ? R1 : R2;
        const int n_strips = (g.OH + R - 1) / R;
        const int blocks = (n_strips * g.OW + 255) / 256;
        if (g.sh == 1)
            hipLaunchKernelGGL((conv_dw3x3_kernel<1, R1>), dim3(blocks, planes), dim3(256), 0, stream, x, wmask, out, g,
                               ep, n_strips);
        else
            hipLaunchKernelGGL((conv_dw3x3_kernel<2, R2>), dim3(blocks, planes), dim3(256), 0, stream, x, wmask, out, g,
                               ep, n_strips);
    } else {
        const int blocks = (g.OH * g.OW + 255) / 256;
        hipLaunchKernelGGL(conv_dw_generic_kernel, dim3(blocks, planes), dim3(256), 0, stream, x, wmask, out, g, ep);
    }
    return hipGetLastError();
}

}  // namespace ohip
