// 3x3 convolution of an image with very few channels (an RGB stem: 3 -> 24 / 32 channels, stride 2), straight from the
// unpacked blob -- fp32 quantized on the way (Tensor/QuantizeX86.cpp:617-641) or int8 -- with no channel-padded copy
// in between. Replaces the reference's pack1to4 path (conv2d_3x3s2_int8_pack1to4_x86 / sgemm pack1to4,
// Tensor/ConvolutionMM2DInt8X86Pack.cpp:148-841) for these shapes.
//
// The reduction is only C*9 <= 45 long, so one v_mfma_i32_16x16x64_i8 holds all of it: B column n is an output pixel,
// its 64 reduction bytes are split over the four lanes (n, kg): lane kg < 3 supplies kernel ROW kg -- the 3 x C input
// values of that row under the window, byte j = 3*c + v -- and lane kg = 3 supplies zeros. A rows are 16 output
// channels with the same byte order (zero where there is no tap). A wave owns 16 consecutive pixels of an output row
// and walks down a strip of rows; per row it gathers and quantizes 3*C values per lane, issues one MFMA per 16 output
// channels and stores 4 channels of its pixel per MFMA (one Float4 element, or half a Byte8 element).
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int STEM_MAX_C = 5;         // 3*C bytes must fit a lane's 16
constexpr int STEM_MAX_TILES = 4;     // K <= 64
constexpr int STEM_ROWS_PER_WAVE = 8;

size_t stem_packed_weight_bytes(int K) { return (size_t)((K + 15) / 16) * 64 * 16; }

// w [K][C][3][3] -> [tile][lane = 16*kg + r][byte j = 3*c + v] = w[16*tile + r][c][kg][v]
void stem_pack_weights(const int8_t* w, int K, int C, int8_t* dst) {
    const int tiles = (K + 15) / 16;
    for (int m = 0; m < tiles; ++m)
        for (int lane = 0; lane < 64; ++lane) {
            const int r = lane & 15, kg = lane >> 4, k = 16 * m + r;
            for (int j = 0; j < 16; ++j) {
                const int c = j / 3, v = j % 3;
                int8_t val = 0;
                if (kg < 3 && c < C && k < K) val = w[(((size_t)k * C + c) * 3 + kg) * 3 + v];
                dst[((size_t)m * 64 + lane) * 16 + j] = val;
            }
        }
}

// CT: the channel count when known at compile time (3: an RGB image), 0: g.C at run time (up to STEM_MAX_C, absent
// channels loaded from a clamped address and dropped)
template <int MT, bool F32_OUT, bool IN_F32, int CT>
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

    constexpr int NC = CT ? CT : STEM_MAX_C;
    const int C = CT ? CT : g.C;
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

// shapes and epilogues this kernel takes; everything else goes through the channel-padded copy and the generic kernel
bool conv_stem_applicable(const ConvGeom& g, const Epilogue& ep, int in_layout) {
    if (g.groups != 1 || g.kh != 3 || g.kw != 3 || g.dh != 1 || g.dw != 1 || g.sh != g.sw || g.sh < 1 || g.sh > 2) return false;
    if (g.ph > 1 || g.pw > 1 || g.C > STEM_MAX_C || g.K > 16 * STEM_MAX_TILES) return false;
    if (in_layout != OTTER_HIP_F32 && in_layout != OTTER_HIP_I8) return false;
    const bool clamp_act = ep.act == 0 || ep.act == 1 || ep.act == 3 || (ep.act == 2 && ep.lrelu);
    if (!clamp_act) return false;
    if (ep.out_kind == OTTER_HIP_OUT_F32) return ep.out_layout == OTTER_HIP_F32_P4 && g.K % 4 == 0;
    if (ep.out_kind == OTTER_HIP_OUT_I8) return ep.out_layout == OTTER_HIP_I8_P8 && g.K % 8 == 0;
    return false;
}

hipError_t run_conv_stem(const void* x, bool in_f32, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const float* in_scale, int in_round, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const int col_groups = (g.OW + 15) / 16;
    const int strips = (g.OH + STEM_ROWS_PER_WAVE - 1) / STEM_ROWS_PER_WAVE;
    const long total = (long)g.N * strips * col_groups;
    if (total >= (1l << 31)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((total + 3) / 4)), block(256);
    const int mt = (g.K + 15) / 16;
    const bool f32_out = ep.out_kind == OTTER_HIP_OUT_F32;
#define OHIP_STEM(MT_, FO_, FI_)                                                                                       \
    do {                                                                                                               \
        if (g.C == 3)                                                                                                  \
            hipLaunchKernelGGL((conv_stem3x3_kernel<MT_, FO_, FI_, 3>), grid, block, 0, stream, x, wpk, out, g, ep,    \
                               in_scale, in_round, col_groups, strips, (int)total);                                    \
        else                                                                                                           \
            hipLaunchKernelGGL((conv_stem3x3_kernel<MT_, FO_, FI_, 0>), grid, block, 0, stream, x, wpk, out, g, ep,    \
                               in_scale, in_round, col_groups, strips, (int)total);                                    \
    } while (0)
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
