// 3x3 convolution of an image with very few channels (an RGB stem: 3 -> 24 / 32 channels, stride 2), straight from the
// unpacked blob -- fp32 quantized on the way (Tensor/QuantizeX86.cpp:617-641) or int8 -- with no channel-padded copy
// in between. Replaces the reference's pack1to4 path (conv2d_3x3s2_int8_pack1to4_x86 / sgemm pack1to4,
// Tensor/ConvolutionMM2DInt8X86Pack.cpp:148-841) for these shapes.
//
// The reduction is only C*9 <= 45 long, so one v_mfma_i32_16x16x64_i8 holds all of it: B column n is an output pixel,
// its 64 reduction bytes are split over the four lanes (n, kg): lane kg < 3 supplies kernel ROW kg -- the 3 x C input
// values of that row under the window -- and lane kg = 3 supplies bytes that meet zero weights. A rows are 16 output
// channels with the same byte order (zero where there is no tap). A wave owns 16 consecutive pixels of an output row;
// per row it issues one MFMA per 16 output channels and stores 4 channels of its pixel per MFMA (one Float4 element,
// or half a Byte8 element).
//
// Up to 4 channels (conv_stem3x3_lds_kernel): a workgroup first quantizes the input rows of a strip of output rows into
// LDS, every value once, with 16-byte loads, as int8 lines [input row][channel][pixel]; a lane's operand is then, per
// channel, the dword that starts at its window's first pixel (two LDS dwords and one v_alignbit): byte 4*c + v, the
// fourth byte of each channel (the next pixel) meeting a zero weight. 5 channels (conv_stem3x3_kernel, byte 3*c + v):
// every lane gathers and quantizes its 3*C values itself.
#include <algorithm>
#include <cstdint>
#include <type_traits>

#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int STEM_MAX_C = 5;         // 3*C bytes must fit a lane's 16
constexpr int STEM_LDS_MAX_C = 4;     // 4*C bytes must fit a lane's 16: the kernel that stages the input in LDS
constexpr int STEM_MAX_TILES = 4;     // K <= 64
constexpr int STEM_ROWS_PER_WAVE = 8;

size_t stem_packed_weight_bytes(int K) { return (size_t)((K + 15) / 16) * 64 * 16; }

// w [K][C][3][3] -> [tile][lane = 16*kg + r][byte j] = w[16*tile + r][c][kg][v], j = 4*c + v for up to 4 channels
// (byte 4*c + 3 stays zero), j = 3*c + v for 5
void stem_pack_weights(const int8_t* w, int K, int C, int8_t* dst) {
    const int tiles = (K + 15) / 16;
    const int per = C <= STEM_LDS_MAX_C ? 4 : 3;
    for (int m = 0; m < tiles; ++m)
        for (int lane = 0; lane < 64; ++lane) {
            const int r = lane & 15, kg = lane >> 4, k = 16 * m + r;
            for (int j = 0; j < 16; ++j) {
                const int c = j / per, v = j % per;
                int8_t val = 0;
                if (kg < 3 && v < 3 && c < C && k < K) val = w[(((size_t)k * C + c) * 3 + kg) * 3 + v];
                dst[((size_t)m * 64 + lane) * 16 + j] = val;
            }
        }
}

// (absent channels are loaded from a clamped address and dropped)
template <int MT, bool F32_OUT, bool IN_F32>
__global__ void __launch_bounds__(256) conv_stem3x3_kernel(const void* __restrict__ x_, const int8_t* __restrict__ wpk,
                                                           void* __restrict__ out, ConvGeom g, Epilogue ep,
                                                           const float* __restrict__ in_scale, int in_round,
                                                           int col_groups, int strips, int total_waves) {
    const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4 + (threadIdx.x >> 6)));
    if (wave >= total_waves) return;
    const int lane = threadIdx.x & 63, n = lane & 15, kg = lane >> 4;
    const int cg = wave % col_groups;
    const int strip = (wave / col_groups) % strips;
    const int img = wave / (col_groups * strips);
    const int ox = cg * 16 + n;
    const int S = g.sh;

    v4i a[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) a[m] = reinterpret_cast<const v4i*>(wpk)[m * 64 + lane];

    // epilogue constants of this lane's channels 16*m + 4*kg + i
    float si[MT][4], bi[MT][4], so[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ch = 16 * m + 4 * kg + i;
            si[m][i] = ep.scale_in[ch];
            bi[m][i] = ep.bias[ch];
            so[m][i] = F32_OUT ? 0.f : ep.scale_out[ch];
        }
    const float qs = IN_F32 ? in_scale[0] : 0.f;
    const float half = in_round == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;

    const int ix0 = ox * S - g.pw;
    const bool col_ok = ox < g.OW;
    const size_t plane = (size_t)g.H * g.W;
    const size_t img_in = (size_t)img * g.C * plane;
    const int OHW = g.OH * g.OW;
    const int oy_end = min((strip + 1) * STEM_ROWS_PER_WAVE, g.OH);

    constexpr int NC = STEM_MAX_C;
    const int C = g.C;
    const unsigned plane_u = (unsigned)plane;
    for (int oy = strip * STEM_ROWS_PER_WAVE; oy < oy_end; ++oy) {
        // ---- this lane's 16 reduction bytes: kernel row kg, byte 3*c + v. Every lane loads all of its 3*NC values
        // from clamped (always valid) addresses first, so that the loads are in flight together; what lies outside
        // the image, the channel count or the kernel is zeroed afterwards.
        const int iy = oy * S - g.ph + kg;
        const bool row_ok = kg < 3 && iy >= 0 && iy < g.H && col_ok;
        const unsigned row_off = (unsigned)min(max(iy, 0), g.H - 1) * (unsigned)g.W;
        unsigned col_off[3];
        bool ok[3];
#pragma unroll
        for (int v = 0; v < 3; ++v) {
            const int ix = ix0 + v;
            ok[v] = row_ok && ix >= 0 && ix < g.W;
            col_off[v] = (unsigned)min(max(ix, 0), g.W - 1);
        }
        float fv[3 * NC];
        int q[15];
#pragma unroll
        for (int j = 0; j < 15; ++j) q[j] = 0;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const unsigned ch_off = (unsigned)min(c, C - 1) * plane_u + row_off;
#pragma unroll
            for (int v = 0; v < 3; ++v) {
                if constexpr (IN_F32) fv[3 * c + v] = static_cast<const float*>(x_)[img_in + ch_off + col_off[v]];
                else q[3 * c + v] = static_cast<const int8_t*>(x_)[img_in + ch_off + col_off[v]];
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int v = 0; v < 3; ++v) {
                if constexpr (IN_F32) {
                    const float t = __fmul_rn(fv[3 * c + v], qs);
                    const int r = (int)__fadd_rn(t, __builtin_copysignf(half, t));
                    q[3 * c + v] = min(max(r, -127), 127);
                }
                if (!(ok[v] && c < C)) q[3 * c + v] = 0;
            }
        v4i b;
        b[0] = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | (q[3] << 24);
        b[1] = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | (q[7] << 24);
        b[2] = (q[8] & 0xff) | ((q[9] & 0xff) << 8) | ((q[10] & 0xff) << 16) | (q[11] << 24);
        b[3] = (q[12] & 0xff) | ((q[13] & 0xff) << 8) | ((q[14] & 0xff) << 16);

        const int pix = oy * g.OW + ox;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[m], b, v4i{0, 0, 0, 0}, 0, 0, 0);
            const int ch0 = 16 * m + 4 * kg;  // D rows 4*kg .. 4*kg+3 of column n
            if (!col_ok || ch0 >= g.K) continue;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float t = __fmaf_rn((float)acc[i], si[m][i], bi[m][i]);
                t = fminf(fmaxf(t, ep.act_lo), ep.act_hi);
                if (ep.lrelu) t = fmaxf(t, __fmul_rn(t, ep.act_p0));
                v[i] = t;
            }
            if constexpr (F32_OUT) {  // Float4: [N][K/4][OH*OW][4]
                float4* o = reinterpret_cast<float4*>(out) + ((size_t)img * (g.K / 4) + ch0 / 4) * OHW + pix;
                *o = make_float4(v[0], v[1], v[2], v[3]);
            } else {  // Byte8: [N][K/8][OH*OW][8]; these 4 channels are one half of an element
                unsigned pk = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float t = __fmul_rn(v[i], so[m][i]);
                    const int r = (int)__fadd_rn(t, __builtin_copysignf(ep.round_half, t));
                    pk |= (unsigned)(min(max(r, -127), 127) & 0xff) << (8 * i);
                }
                unsigned* o = reinterpret_cast<unsigned*>(out) + (((size_t)img * (g.K / 8) + ch0 / 8) * OHW + pix) * 2 + (ch0 / 4 & 1);
                *o = pk;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// Up to 4 channels: the strip's input rows quantized into LDS once, operands from LDS
// ---------------------------------------------------------------------------------------------------------------------

// A workgroup (4 waves) owns R output rows of one image. LDS: [input row r < RIN][channel][pitch_dw dwords] of int8;
// dword d of a line holds pixels 4*(d-1) .. 4*(d-1)+3 (dword 0 and everything past the row's end are zeros: the
// padding columns), rows outside the image are zeros.
struct StemPlan {
    int R, strips, cgs, RIN, pitch_dw, vec;
    float inv_pitch, inv_c;
};

constexpr int STEM_UN = 8;        // 4-pixel units a thread has in flight while the strip is loaded
constexpr int STEM_LDS_ROWS = 4;  // output rows per workgroup (measured: 2, 4, 8 within 5 % of each other at 224 x 224, 16 slower)

// EPI: 0 = fp32 Float4 result, 1 = int8 Byte8, 2 = int8 Byte8 of a layer that clamps at zero with positive output
// scales (the clamp applied to the rounded values, see epi8_quant_i8p8)
template <int MT, int EPI, bool IN_F32, int CT>
__global__ void __launch_bounds__(256) conv_stem3x3_lds_kernel(const void* __restrict__ x_, const int8_t* __restrict__ wpk,
                                                               void* __restrict__ out, ConvGeom g, Epilogue ep,
                                                               const float* __restrict__ in_scale, int in_round, StemPlan p) {
    extern __shared__ unsigned stem_lds[];
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int img = (int)blockIdx.x / p.strips, strip = (int)blockIdx.x - img * p.strips;
    const int S = g.sh, C = CT ? CT : g.C;
    constexpr int NC = CT ? CT : STEM_LDS_MAX_C;

    // ---- the strip's input rows -> int8 lines in LDS
    const int oy0 = strip * p.R, iy0 = oy0 * S - g.ph;
    const int total = p.RIN * C * p.pitch_dw;
    const unsigned plane = (unsigned)(g.H * g.W);
    const size_t img_in = (size_t)img * g.C * plane;
    const float qs = IN_F32 ? in_scale[0] : 0.f;
    const float half = in_round == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
    auto fill = [&](auto vec_tag) {
        constexpr bool VEC = decltype(vec_tag)::value;  // rows of whole, aligned 4-pixel units: one load per unit
        for (int base = 0; base < total; base += 256 * STEM_UN) {
            v4i raw[STEM_UN];
            unsigned keep[STEM_UN];
#pragma unroll
            for (int j = 0; j < STEM_UN; ++j) {
                if (base + 256 * j + 64 * wave >= total) continue;  // (none of this wave's units exists)
                // unit idx = dword idx of the LDS image: line = idx / pitch, row = line / C (exact: the quotients' fractional
                // parts stay 0.5 / divisor away from an integer, far more than the rounding of these products)
                const int idx = min(base + 256 * j + tid, total - 1);
                const int line = (int)(((float)idx + 0.5f) * p.inv_pitch);
                const int d = idx - line * p.pitch_dw;
                const int r = (int)(((float)line + 0.5f) * p.inv_c);
                const int c = line - r * C;
                const int iy = iy0 + r, ix = 4 * (d - 1);
                const bool row_ok = iy >= 0 && iy < g.H;
                const unsigned off0 = (unsigned)c * plane + (unsigned)min(max(iy, 0), g.H - 1) * (unsigned)g.W;
                // every load from a clamped (always valid) address, so that all are in flight together; what lies outside
                // the image is zeroed afterwards
                if constexpr (VEC) {
                    const unsigned off = off0 + (unsigned)min(max(ix, 0), g.W - 4);
                    if constexpr (IN_F32) raw[j] = *reinterpret_cast<const v4i*>(static_cast<const float*>(x_) + img_in + off);
                    else raw[j][0] = *reinterpret_cast<const int*>(static_cast<const int8_t*>(x_) + img_in + off);
                    keep[j] = row_ok && ix >= 0 && ix < g.W ? 0xffffffffu : 0u;
                } else {
                    unsigned k = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int ixe = ix + e;
                        const unsigned off = off0 + (unsigned)min(max(ixe, 0), g.W - 1);
                        if constexpr (IN_F32) raw[j][e] = __float_as_int(static_cast<const float*>(x_)[img_in + off]);
                        else raw[j][e] = static_cast<const int8_t*>(x_)[img_in + off];
                        if (row_ok && ixe >= 0 && ixe < g.W) k |= 0xffu << (8 * e);
                    }
                    keep[j] = k;
                }
            }
#pragma unroll
            for (int j = 0; j < STEM_UN; ++j) {
                if (base + 256 * j + 64 * wave >= total) continue;
                unsigned pk;
                if constexpr (IN_F32) {
                    int q[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float t = __fmul_rn(__int_as_float(raw[j][e]), qs);
                        q[e] = (int)__fadd_rn(t, __builtin_copysignf(half, t));
                    }
                    const ohip_v2s top = {127, 127}, bot = {-127, -127};
                    ohip_v2s lo = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[0], q[1]));
                    ohip_v2s hi = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[2], q[3]));
                    lo = __builtin_elementwise_max(__builtin_elementwise_min(lo, top), bot);
                    hi = __builtin_elementwise_max(__builtin_elementwise_min(hi, top), bot);
                    pk = __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
                } else if constexpr (VEC) {
                    pk = (unsigned)raw[j][0];
                } else {
                    pk = (unsigned)(raw[j][0] & 0xff) | (unsigned)(raw[j][1] & 0xff) << 8 | (unsigned)(raw[j][2] & 0xff) << 16 |
                         (unsigned)raw[j][3] << 24;
                }
                const int idx = base + 256 * j + tid;
                if (idx < total) stem_lds[idx] = pk & keep[j];
            }
        }
    };
    if (p.vec) fill(std::true_type{});
    else fill(std::false_type{});

    // ---- this lane's weights and the constants of its channels 16*m + 4*kg + i (requested once the strip's loads have
    // been consumed, so that their registers are not held across them; they arrive while the workgroup meets at the barrier)
    v4i a[MT];
    float si[MT][4], bi[MT][4], so[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        a[m] = reinterpret_cast<const v4i*>(wpk)[m * 64 + lane];
        const int ch = 16 * m + 4 * kg;
        const v4i s4 = *reinterpret_cast<const v4i*>(ep.scale_in + ch), b4 = *reinterpret_cast<const v4i*>(ep.bias + ch);
        v4i o4 = {0, 0, 0, 0};
        if constexpr (EPI != 0) o4 = *reinterpret_cast<const v4i*>(ep.scale_out + ch);
#pragma unroll
        for (int i = 0; i < 4; ++i) si[m][i] = __int_as_float(s4[i]), bi[m][i] = __int_as_float(b4[i]), so[m][i] = __int_as_float(o4[i]);
    }

    unsigned qh[MT][2];
    if constexpr (EPI == 2) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            qh[m][0] = epi8_clamp_pair(ep, so[m][0], so[m][1]);
            qh[m][1] = epi8_clamp_pair(ep, so[m][2], so[m][3]);
        }
    }
    __syncthreads();

    // ---- the output rows of the strip: item = (row, group of 16 pixels)
    const int rows = min(p.R, g.OH - oy0);
    const int items = rows * p.cgs;
    const int lc0 = S * n - g.pw + 4;  // this lane's window starts at this byte of a line (plus 16*S per pixel group)
    const unsigned shift = 8u * (unsigned)(lc0 & 3);
    const int OHW = g.OH * g.OW;
    for (int it = wave; it < items; it += 4) {
        const int orow = it / p.cgs, cg = it - orow * p.cgs;
        const int r = min(S * orow + kg, p.RIN - 1);  // (kernel row 3 does not exist: its bytes meet zero weights)
        const unsigned* line = stem_lds + r * C * p.pitch_dw + (lc0 >> 2) + 4 * S * cg;
        v4i b = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const unsigned* l = line + (CT ? c : min(c, C - 1)) * p.pitch_dw;  // (absent channels meet zero weights too)
            b[c] = (int)__builtin_amdgcn_alignbit(l[1], l[0], shift);
        }
        const int ox = 16 * cg + n;
        const bool col_ok = ox < g.OW;
        const int pix = (oy0 + orow) * g.OW + ox;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[m], b, v4i{0, 0, 0, 0}, 0, 0, 0);
            const int ch0 = 16 * m + 4 * kg;  // D rows 4*kg .. 4*kg+3 of column n
            if (!col_ok || ch0 >= g.K) continue;
            if constexpr (EPI == 2) {
                int q[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float t = __fmul_rn(__fmaf_rn((float)acc[i], si[m][i], bi[m][i]), so[m][i]);
                    q[i] = (int)cvt_u32_floor0(__fadd_rn(t, ep.round_half));  // (to unsigned: the clamp at zero comes with it)
                }
                typedef unsigned short ohip_v2us __attribute__((ext_vector_type(2)));
                ohip_v2us lo = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)q[0], (unsigned)q[1]));
                ohip_v2us hi = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)q[2], (unsigned)q[3]));
                lo = __builtin_elementwise_min(lo, __builtin_bit_cast(ohip_v2us, qh[m][0]));
                hi = __builtin_elementwise_min(hi, __builtin_bit_cast(ohip_v2us, qh[m][1]));
                unsigned* o = reinterpret_cast<unsigned*>(out) + (((size_t)img * (g.K / 8) + ch0 / 8) * OHW + pix) * 2 + (ch0 / 4 & 1);
                *o = __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
            } else {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float t = __fmaf_rn((float)acc[i], si[m][i], bi[m][i]);
                    t = fminf(fmaxf(t, ep.act_lo), ep.act_hi);
                    if (ep.lrelu) t = fmaxf(t, __fmul_rn(t, ep.act_p0));
                    v[i] = t;
                }
                if constexpr (EPI == 0) {  // Float4: [N][K/4][OH*OW][4]
                    float4* o = reinterpret_cast<float4*>(out) + ((size_t)img * (g.K / 4) + ch0 / 4) * OHW + pix;
                    *o = make_float4(v[0], v[1], v[2], v[3]);
                } else {  // Byte8: [N][K/8][OH*OW][8]; these 4 channels are one half of an element
                    unsigned pk = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float t = __fmul_rn(v[i], so[m][i]);
                        const int rr = (int)__fadd_rn(t, __builtin_copysignf(ep.round_half, t));
                        pk |= (unsigned)(min(max(rr, -127), 127) & 0xff) << (8 * i);
                    }
                    unsigned* o = reinterpret_cast<unsigned*>(out) + (((size_t)img * (g.K / 8) + ch0 / 8) * OHW + pix) * 2 + (ch0 / 4 & 1);
                    *o = pk;
                }
            }
        }
    }
}

// rows per workgroup and the LDS image of a strip; false where even one output row's input does not fit 64 KB
static bool stem_lds_plan(const ConvGeom& g, StemPlan* p, size_t* lds_bytes) {
    const int S = g.sh, cgs = (g.OW + 15) / 16;
    const int pitch_dw = std::max(((S * (16 * cgs - 1) - g.pw + 4) >> 2) + 2, (g.W + 3) / 4 + 1);
    for (int R = std::min(STEM_LDS_ROWS, g.OH); R >= 1; --R) {
        const int RIN = S * (R - 1) + 3;
        const size_t bytes = (size_t)RIN * g.C * pitch_dw * 4;
        if (bytes > 64 * 1024) continue;
        p->R = R, p->strips = (g.OH + R - 1) / R, p->cgs = cgs, p->RIN = RIN, p->pitch_dw = pitch_dw, p->vec = 0;
        p->inv_pitch = 1.0f / (float)pitch_dw, p->inv_c = 1.0f / (float)g.C;
        *lds_bytes = bytes;
        return true;
    }
    return false;
}

// shapes and epilogues this kernel takes; everything else goes through the channel-padded copy and the generic kernel
bool conv_stem_applicable(const ConvGeom& g, const Epilogue& ep, int in_layout) {
    if (g.groups != 1 || g.kh != 3 || g.kw != 3 || g.dh != 1 || g.dw != 1 || g.sh != g.sw || g.sh < 1 || g.sh > 2) return false;
    if (g.ph > 1 || g.pw > 1 || g.C > STEM_MAX_C || g.K > 16 * STEM_MAX_TILES) return false;
    if (in_layout != OTTER_HIP_F32 && in_layout != OTTER_HIP_I8) return false;
    if (g.C <= STEM_LDS_MAX_C) {  // (the weights are packed for the kernel that stages the input in LDS)
        StemPlan p;
        size_t lds = 0;
        if ((long)g.C * g.H * g.W >= (1l << 31) || !stem_lds_plan(g, &p, &lds)) return false;
    }
    const bool clamp_act = ep.act == 0 || ep.act == 1 || ep.act == 3 || (ep.act == 2 && ep.lrelu);
    if (!clamp_act) return false;
    if (ep.out_kind == OTTER_HIP_OUT_F32) return ep.out_layout == OTTER_HIP_F32_P4 && g.K % 4 == 0;
    if (ep.out_kind == OTTER_HIP_OUT_I8) return ep.out_layout == OTTER_HIP_I8_P8 && g.K % 8 == 0;
    return false;
}

template <int MT>
static hipError_t launch_stem_lds(const void* x, bool in_f32, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                  const float* in_scale, int in_round, hipStream_t stream) {
    StemPlan p;
    size_t lds = 0;
    if (!stem_lds_plan(g, &p, &lds)) return hipErrorInvalidValue;
    const long wgs = (long)g.N * p.strips;
    if (wgs >= (1l << 31)) return hipErrorInvalidValue;
    // whole 4-pixel units at aligned addresses: one 16-byte (fp32) or 4-byte (int8) load per unit
    p.vec = g.W % 4 == 0 && ((uintptr_t)x & (in_f32 ? 15 : 3)) == 0;
    const int epi = ep.out_kind == OTTER_HIP_OUT_F32 ? 0 : pick_epilogue(ep, g.K) == EPI_I8_P8_NONNEG ? 2 : 1;
    const dim3 grid((unsigned)wgs), block(256);
#define OHIP_STEM_L(EPI_, FI_)                                                                                          \
    do {                                                                                                                \
        if (g.C == 3)                                                                                                   \
            hipLaunchKernelGGL((conv_stem3x3_lds_kernel<MT, EPI_, FI_, 3>), grid, block, lds, stream, x, wpk, out, g, ep, \
                               in_scale, in_round, p);                                                                  \
        else                                                                                                            \
            hipLaunchKernelGGL((conv_stem3x3_lds_kernel<MT, EPI_, FI_, 0>), grid, block, lds, stream, x, wpk, out, g, ep, \
                               in_scale, in_round, p);                                                                  \
    } while (0)
    if (in_f32) {
        if (epi == 0) OHIP_STEM_L(0, true);
        else if (epi == 1) OHIP_STEM_L(1, true);
        else OHIP_STEM_L(2, true);
    } else {
        if (epi == 0) OHIP_STEM_L(0, false);
        else if (epi == 1) OHIP_STEM_L(1, false);
        else OHIP_STEM_L(2, false);
    }
#undef OHIP_STEM_L
    return hipGetLastError();
}

hipError_t run_conv_stem(const void* x, bool in_f32, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const float* in_scale, int in_round, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const int mt = (g.K + 15) / 16;
    if (g.C <= STEM_LDS_MAX_C) {
        switch (mt) {
        case 1: return launch_stem_lds<1>(x, in_f32, wpk, out, g, ep, in_scale, in_round, stream);
        case 2: return launch_stem_lds<2>(x, in_f32, wpk, out, g, ep, in_scale, in_round, stream);
        case 3: return launch_stem_lds<3>(x, in_f32, wpk, out, g, ep, in_scale, in_round, stream);
        case 4: return launch_stem_lds<4>(x, in_f32, wpk, out, g, ep, in_scale, in_round, stream);
        default: return hipErrorInvalidValue;
        }
    }
    const int col_groups = (g.OW + 15) / 16;
    const int strips = (g.OH + STEM_ROWS_PER_WAVE - 1) / STEM_ROWS_PER_WAVE;
    const long total = (long)g.N * strips * col_groups;
    if (total >= (1l << 31)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((total + 3) / 4)), block(256);
    const bool f32_out = ep.out_kind == OTTER_HIP_OUT_F32;
#define OHIP_STEM(MT_, FO_, FI_)                                                                                   \
    hipLaunchKernelGGL((conv_stem3x3_kernel<MT_, FO_, FI_>), grid, block, 0, stream, x, wpk, out, g, ep, in_scale,    \
                       in_round, col_groups, strips, (int)total)
#define OHIP_STEM_IO(MT_)                                  \
    do {                                                   \
        if (f32_out && in_f32) OHIP_STEM(MT_, true, true); \
        else if (f32_out) OHIP_STEM(MT_, true, false);     \
        else if (in_f32) OHIP_STEM(MT_, false, true);      \
        else OHIP_STEM(MT_, false, false);                 \
    } while (0)
    switch (mt) {
    case 1: OHIP_STEM_IO(1); break;
    case 2: OHIP_STEM_IO(2); break;
    case 3: OHIP_STEM_IO(3); break;
    case 4: OHIP_STEM_IO(4); break;
    default: return hipErrorInvalidValue;
    }
#undef OHIP_STEM_IO
#undef OHIP_STEM
    return hipGetLastError();
}

}  // namespace ohip
