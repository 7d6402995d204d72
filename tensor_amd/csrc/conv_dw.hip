// Depthwise int8 convolution on the reference's Byte8 layout: a bandwidth-bound kernel, no MFMA.
//
// One (image, channel octet) plane [H, W, 8 bytes] is independent of every other, so a workgroup works inside
// one plane: its 8 x maxk weights and its 8 scale/bias values are wave-uniform and live in scalar registers.
// A lane owns one output column and walks down a strip of output rows, so consecutive lanes read consecutive
// 8-byte pixels (a wave reads 512 contiguous bytes per tap column) and every input row is fetched once per
// strip and reused from registers for the rows below it.
// The multiply-accumulate uses v_dot4_i32_i8 against a weight word that holds the tap weight in the byte of
// its channel and zeros elsewhere: one instruction per (tap, channel) with no byte unpacking of the input.
#include <algorithm>

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

// first tap: the three-operand form with a literal zero accumulator (the compiler would otherwise emit a zeroing
// move plus the accumulate-in-place form for every output)
__device__ __forceinline__ int dot4_first(int x, int w) {
    int r;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(x), "s"(w));
    return r;
}

__device__ __forceinline__ void mac8(int (&acc)[8], v2i px, const int* __restrict__ wm) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = __builtin_amdgcn_sdot4(px[0], wm[e], acc[e], false);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[4 + e] = __builtin_amdgcn_sdot4(px[1], wm[4 + e], acc[4 + e], false);
}

// 3x3, dilation 1, stride S (1 or 2): R output rows per lane with the input rows kept in registers.
template <int S, int R, int EPI>
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
    // per-channel epilogue constants: wave-uniform (one channel octet per workgroup), so they sit in SGPRs
    Epi8 prm;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        prm.si[e] = ep.scale_in[o * 8 + e];
        prm.bi[e] = ep.bias[o * 8 + e];
        prm.so[e] = ep.scale_out ? ep.scale_out[o * 8 + e] : 1.f;
    }
    if constexpr (EPI == EPI_I8_P8_NONNEG) epi8_clamp_init(ep, prm);

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
        const int pix = oy * g.OW + ox;
        if constexpr (EPI == EPI_I8_P8 || EPI == EPI_I8_P8_NONNEG) {
            epi8_store_i8p8<EPI == EPI_I8_P8_NONNEG>((int8_t*)out, ep, prm, ((size_t)plane * OHW + pix) * 8, acc);
        } else {
            epilogue_store8(out, ep, n, o * 8, pix, g.K, OHW, acc, prm.si, prm.bi, prm.so);
        }
    }
}

// 3x3, int8 Byte8 out (the requantize epilogue): same strip walk, but the channel octet is processed as two
// halves of four channels, one after the other. A half needs 36 weight words + 12 epilogue constants, which fit
// the scalar register file; the whole octet (72 + 24) does not, and spilling them to VGPR lanes costs more VALU
// work than the convolution itself. The first tap starts the accumulator (no zero-initialisation moves).
template <int S, int R, bool NONNEG>
__global__ void __launch_bounds__(256) conv_dw3x3_i8_kernel(const int8_t* __restrict__ x, const int32_t* __restrict__ wmask,
                                                            int8_t* __restrict__ out, ConvGeom g, Epilogue ep,
                                                            int n_strips, int col_chunks, int ipw) {
    // A wave = 64 consecutive output columns of ONE strip, so "is this input row inside the image" is a scalar
    // branch, not a per-lane exec mask (those masks would crowd the weights out of the scalar registers).
    // Images narrower than half a wave put `ipw` images side by side in the wave instead (same channel octet, same
    // strip, consecutive images): the weights and the row test stay wave-uniform and the lanes stay busy.
    const int C8 = g.C / 8;
    const int o = blockIdx.y % C8;
    const int n0 = (blockIdx.y / C8) * ipw;
    const int chunk = blockIdx.x % col_chunks;
    const int strip = __builtin_amdgcn_readfirstlane((blockIdx.x / col_chunks) * (blockDim.x >> 6) + (threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    int di = 0, ox = chunk * 64 + lane;
    if (ipw > 1) {
        di = lane / g.OW;
        ox = lane - di * g.OW;
    }
    if (strip >= n_strips || ox >= g.OW || di >= ipw || n0 + di >= g.N) return;

    // scalar base of the wave's first image + a 32-bit lane offset (the host keeps ipw image strides below 2^31)
    const int8_t* xp = x + ((size_t)n0 * C8 + o) * g.H * g.W * 8;
    const unsigned in_img = (unsigned)di * (unsigned)(C8 * g.H * g.W * 8);
    const int ix0 = ox * S - g.pw;
    // columns 0 and 2 of the window can fall off the image for the first / last output column only: read a clamped
    // address and zero the value
    // (the middle column is always inside: pad <= 1 is checked on the host)
    const bool c0_ok = ix0 >= 0, c2_ok = ix0 + 2 < g.W;
    const unsigned ixc0 = in_img + max(ix0, 0) * 8, ixc1 = in_img + (ix0 + 1) * 8, ixc2 = in_img + min(ix0 + 2, g.W - 1) * 8;
    const int oy0 = strip * R;
    const int OHW = g.OH * g.OW;

    constexpr int NROWS = (R - 1) * S + 3;  // input rows a strip touches
    v2i rows[NROWS][3];
    const int iy_base = oy0 * S - g.ph;
#pragma unroll
    for (int r = 0; r < NROWS; ++r) {
        const int iy = iy_base + r;
        if (iy >= 0 && iy < g.H) {  // wave-uniform
            const int8_t* rp = xp + (size_t)iy * g.W * 8;
            const v2i a = *reinterpret_cast<const v2i*>(rp + ixc0);
            const v2i b = *reinterpret_cast<const v2i*>(rp + ixc1);
            const v2i c = *reinterpret_cast<const v2i*>(rp + ixc2);
            rows[r][0] = c0_ok ? a : v2i{0, 0};
            rows[r][1] = b;
            rows[r][2] = c2_ok ? c : v2i{0, 0};
        } else {
            rows[r][0] = rows[r][1] = rows[r][2] = v2i{0, 0};
        }
    }

    int packed[2][R];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        int wm[9][4];
        float si[4], bi[4], so[4];
        const int* wsrc = wmask + (size_t)o * 72 + h * 4;
#pragma unroll
        for (int k = 0; k < 9; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) wm[k][e] = wsrc[k * 8 + e];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            si[e] = ep.scale_in[o * 8 + h * 4 + e];
            // the bias lives in a vector register: fma(acc, scale, bias) may name only one scalar operand
            asm volatile("v_mov_b32 %0, %1" : "=v"(bi[e]) : "s"(ep.bias[o * 8 + h * 4 + e]));
            so[e] = ep.scale_out[o * 8 + h * 4 + e];
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int acc = dot4_first(rows[r * S][0][h], wm[0][e]);
#pragma unroll
                for (int k = 1; k < 9; ++k) acc = __builtin_amdgcn_sdot4(rows[r * S + k / 3][k % 3][h], wm[k][e], acc, false);
                float v = __fmaf_rn((float)acc, si[e], bi[e]);
                v = __builtin_amdgcn_fmed3f(v, ep.act_lo, ep.act_hi);
                if (!NONNEG && ep.lrelu) v = fmaxf(v, __fmul_rn(v, ep.act_p0));  // wave-uniform branch
                v = __fmul_rn(v, so[e]);
                const float adj =
                    NONNEG ? __fadd_rn(v, ep.round_half) : __fadd_rn(v, __builtin_copysignf(ep.round_half, v));
                q[e] = (int)adj;
            }
            ohip_v2s lo = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[0], q[1]));
            ohip_v2s hi = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[2], q[3]));
            const ohip_v2s top = {127, 127}, bot = {-127, -127};
            lo = __builtin_elementwise_min(lo, top);
            hi = __builtin_elementwise_min(hi, top);
            if (!NONNEG) {
                lo = __builtin_elementwise_max(lo, bot);
                hi = __builtin_elementwise_max(hi, bot);
            }
            packed[h][r] =
                (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
        }
        __builtin_amdgcn_sched_barrier(0);  // the second half's scalars are fetched after the first half is done
    }
    int8_t* op = out + ((size_t)n0 * C8 + o) * OHW * 8;
    const unsigned out_lane = (unsigned)di * (unsigned)(C8 * OHW * 8) + (unsigned)ox * 8;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int oy = oy0 + r;
        if (oy < g.OH) *reinterpret_cast<v2i*>(op + (size_t)oy * g.OW * 8 + out_lane) = v2i{packed[0][r], packed[1][r]};
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
                       int strip_shift, hipStream_t stream) {
    const int planes = g.N * (g.C / 8);
    if (planes == 0 || g.OH * g.OW == 0) return hipSuccess;
    if (planes > 65535) return hipErrorInvalidValue;  // grid.y limit; the caller splits the batch
    const bool k3 = g.kh == 3 && g.kw == 3 && g.dh == 1 && g.dw == 1 && g.sh == g.sw && (g.sh == 1 || g.sh == 2);
    if (k3) {
        constexpr int R1 = 8, R2 = 4;
        const int R = g.sh == 1 ? R1 : R2;
        const int n_strips = (g.OH + R - 1) / R;
        const int blocks = (n_strips * g.OW + 255) / 256;
        int epi = pick_epilogue(ep, g.K);
        if (g.pw > 1 || g.ph > 1) epi = EPI_GENERIC;  // the fast kernel assumes the window's middle column is inside
#define OHIP_DW(S_, R_, E_) \
    hipLaunchKernelGGL((conv_dw3x3_kernel<S_, R_, E_>), dim3(blocks, planes), dim3(256), 0, stream, x, wmask, out, g, ep, \
                       n_strips)
        // narrow images: several images of the same channel octet share a wave (lane offsets stay below 2^31)
        const int col_chunks = (g.OW + 63) / 64;
        int ipw = 1;
        if (g.OW <= 32) {
            ipw = std::min(64 / g.OW, g.N);
            const size_t img = (size_t)g.C * std::max(g.H * g.W, g.OH * g.OW);
            while (ipw > 1 && img * ipw >= ((size_t)1 << 31)) --ipw;
        }
        const int groups8 = ((g.N + ipw - 1) / ipw) * (g.C / 8);
        // rows per strip: the tallest strip (most reuse of input rows, fewest scalar loads per output) that still gives
        // every SIMD four waves; a small layer is latency-bound and wants many short waves instead
        int shift = 0;  // strip height = R >> shift
        if (strip_shift >= 0) shift = std::min(strip_shift, 2);
        else while (shift < 2 && (long)col_chunks * ((g.OH + (R >> shift) - 1) / (R >> shift)) * groups8 < 4096) ++shift;
        const int Rs = R >> shift;
        const int strips8 = (g.OH + Rs - 1) / Rs;
        // one wave per (strip, 64-column chunk); waves per workgroup chosen so that no wave is born idle
        const int wpb = strips8 % 4 == 0 ? 4 : (strips8 % 2 == 0 ? 2 : 1);
        const int blocks8 = col_chunks * (strips8 / wpb);
#define OHIP_DW8(S_, R_, N_) \
    hipLaunchKernelGGL((conv_dw3x3_i8_kernel<S_, R_, N_>), dim3(blocks8, groups8), dim3(64 * wpb), 0, stream, x, wmask, \
                       (int8_t*)out, g, ep, strips8, col_chunks, ipw)
#define OHIP_DW8_R(S_, RMAX_, N_)                  \
    do {                                           \
        if (shift == 0) OHIP_DW8(S_, RMAX_, N_);   \
        else if (shift == 1) OHIP_DW8(S_, RMAX_ / 2, N_); \
        else OHIP_DW8(S_, RMAX_ / 4, N_);          \
    } while (0)
        if (g.sh == 1) {
            if (epi == EPI_I8_P8_NONNEG) OHIP_DW8_R(1, R1, true);
            else if (epi == EPI_I8_P8) OHIP_DW8_R(1, R1, false);
            else OHIP_DW(1, R1, EPI_GENERIC);
        } else {
            if (epi == EPI_I8_P8_NONNEG) OHIP_DW8_R(2, R2, true);
            else if (epi == EPI_I8_P8) OHIP_DW8_R(2, R2, false);
            else OHIP_DW(2, R2, EPI_GENERIC);
        }
#undef OHIP_DW8_R
#undef OHIP_DW
#undef OHIP_DW8
    } else {
        const int blocks = (g.OH * g.OW + 255) / 256;
        hipLaunchKernelGGL(conv_dw_generic_kernel, dim3(blocks, planes), dim3(256), 0, stream, x, wmask, out, g, ep);
    }
    return hipGetLastError();
}

}  // namespace ohip
