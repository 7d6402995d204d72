// Pointwise (1x1, stride 1) int8 -> int8 convolution over at most 64 input channels, or 200 .. 256 on large blobs, as a
// streaming kernel.
//
// With one (or, on large blobs, four) MFMA reduction steps per output the layer is an elementwise pass: read C bytes per pixel, write K
// bytes, and the time goes into the requantization of the K results, not into the product. The implicit-GEMM kernel pays
// for its generality here (output rows padded to its row tile, the pixels' round trip through LDS and two barriers
// per workgroup for one MFMA step, a workgroup prologue per tile). This kernel has no tile grid and one barrier:
//   - a wave owns G groups of 16 consecutive pixels of one image and loads their bytes straight into the MFMA's
//     B operands (reduction step cg, lane (q, p): channels 64cg+16q..+15 of pixel p = two 8-byte elements of the
//     Byte8 blob);
//   - it walks the output channels in pairs of 16-row tiles (32 channels); the A operands (the implicit-GEMM weight
//     packing as it lies in memory, 16 bytes per lane and tile) and the per-channel constants of the workgroup's
//     pairs sit in LDS, copied there once per workgroup, and are read once per pair for all G groups;
//   - after the two MFMAs of a pair each lane holds 8 consecutive output channels of one pixel (the row
//     permutation of igemm_row_channel), requantizes them and stores one Byte8 element: 16 lanes cover 128
//     contiguous bytes.
// Only whole channel octets are stored, so K need not be a multiple of 32; the padded rows cost their MFMA only.
#include "common.hpp"
#include "conv_igemm.hpp"

#include <algorithm>

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v2u_store __attribute__((__vector_size__(2 * sizeof(unsigned))));

constexpr unsigned PW_OOB = 0x80000000u;  // past any buffer: the load returns zero, the store is dropped

// LDS image of one pair of row tiles: per reduction step the two A operands in lane order, then scale_in, bias,
// scale_out (32 floats each) and the clamps (16 dwords) of the pair's 32 channels
constexpr int pw_pair_v4(int cg) { return 128 * cg + 8 + 8 + 8 + 4; }  // 16-byte units
constexpr int pw_max_pairs(int cg) { return (64 * 1024) / (pw_pair_v4(cg) * 16); }  // a slice's image stays under 64 KB
constexpr int PW_MAX_CG = 4;

// grid: x = chunks of 4 waves x G groups x 16 pixels of an image, y = image, z = slice of the channel pairs
// qh (EPI_I8_P8_NONNEG): the upper clamps of the rounded results, one 16-bit value per padded channel
// (conv_pw_stream_clamps)
// The four waves of a workgroup share one copy of their slice's weights and constants in LDS: read from there a
// lane group's constants are one broadcast each, where 64 lanes loading them from memory keep the texture
// addresser busy for longer than the requantization of two pixel groups takes.
// CG: reduction steps (64 input channels each); mt: 16-row tiles of the packed weights per reduction step
template <int EPI, int G, int CG>
__global__ void __launch_bounds__(256) conv_pw_stream_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk,
                                                             int8_t* __restrict__ out, Epilogue ep,
                                                             const unsigned* __restrict__ qh, int C8, int K, int HW,
                                                             int pairs_per_slice, int mt) {
    constexpr int PW_PAIR_V4 = pw_pair_v4(CG);
    extern __shared__ v4i pw_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane >> 4, p = lane & 15;
    const int n = blockIdx.y;
    const int pix0 = (blockIdx.x * 4 + wave) * (16 * G);

    const size_t in_img = (size_t)C8 * HW * 8, out_img = (size_t)K * HW;
    const __amdgpu_buffer_rsrc_t rin =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(x) + (size_t)n * in_img, 0, (int)in_img, 0x00020000);
    const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(out + (size_t)n * out_img, 0, (int)out_img, 0x00020000);

    // B operands of the G groups (all out of range for a wave past the image: zeros, and nothing is stored)
    v4i b[G][CG];
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
        const int pix = pix0 + 16 * gi + p;
        const bool in = pix < HW;
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            const int oct = 8 * cg + 2 * q;
            const unsigned o0 = ((unsigned)oct * HW + pix) * 8u;
            const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(in && oct < C8 ? o0 : PW_OOB), 0, 0));
            const v2i hi = __builtin_bit_cast(
                v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(in && oct + 1 < C8 ? o0 + (unsigned)HW * 8u : PW_OOB), 0, 0));
            b[gi][cg] = v4i{lo[0], lo[1], hi[0], hi[1]};
        }
    }

    const int pairs = (K + 31) / 32;
    const int pr0 = blockIdx.z * pairs_per_slice;
    const int pr1 = min(pr0 + pairs_per_slice, pairs);
    {
        // the per-channel arrays are padded to the weight rows, so every pair is whole in memory
        const v4i* wg = reinterpret_cast<const v4i*>(wpk);
        const v4i* sg = reinterpret_cast<const v4i*>(ep.scale_in);
        const v4i* bg = reinterpret_cast<const v4i*>(ep.bias);
        const v4i* og = reinterpret_cast<const v4i*>(ep.scale_out);
        const v4i* cg = reinterpret_cast<const v4i*>(qh);
        const int total = (pr1 - pr0) * PW_PAIR_V4;
        for (int i = threadIdx.x; i < total; i += 256) {
            const int pr = pr0 + i / PW_PAIR_V4, r = i % PW_PAIR_V4;
            constexpr int W4 = 128 * CG;
            v4i v;
            if (r < W4) v = wg[((size_t)(r / 128) * mt + 2 * pr) * 64 + r % 128];  // (step, the pair's two tiles, lane)
            else if (r < W4 + 8) v = sg[pr * 8 + r - W4];
            else if (r < W4 + 16) v = bg[pr * 8 + r - W4 - 8];
            else if (r < W4 + 24) v = og[pr * 8 + r - W4 - 16];
            else if constexpr (EPI == EPI_I8_P8_NONNEG) v = cg[pr * 4 + r - W4 - 24];
            else v = v4i{0, 0, 0, 0};
            pw_lds[i] = v;
        }
    }
    __syncthreads();
    if (pix0 >= HW) return;

    for (int pr = pr0; pr < pr1; ++pr) {
        const v4i* l = pw_lds + (pr - pr0) * PW_PAIR_V4;
        v4i a0[CG], a1[CG];
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) a0[cg] = l[128 * cg + lane], a1[cg] = l[128 * cg + 64 + lane];
        Epi8 prm;
        {
            constexpr int W4 = 128 * CG;
            const v4i s0 = l[W4 + 2 * q], s1 = l[W4 + 1 + 2 * q], b0 = l[W4 + 8 + 2 * q], b1 = l[W4 + 9 + 2 * q];
            const v4i o0 = l[W4 + 16 + 2 * q], o1 = l[W4 + 17 + 2 * q], c = l[W4 + 24 + q];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                prm.si[e] = __int_as_float(s0[e]), prm.si[4 + e] = __int_as_float(s1[e]);
                prm.bi[e] = __int_as_float(b0[e]), prm.bi[4 + e] = __int_as_float(b1[e]);
                prm.so[e] = __int_as_float(o0[e]), prm.so[4 + e] = __int_as_float(o1[e]);
                prm.qh[e] = (unsigned)c[e];
            }
        }
        const int ch0 = 32 * pr + 8 * q;
        const bool live = ch0 < K;
        const unsigned orow = (unsigned)(ch0 >> 3) * HW;
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
            v4i c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[0], b[gi][0], v4i{0, 0, 0, 0}, 0, 0, 0);
            v4i c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[0], b[gi][0], v4i{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
            for (int cg = 1; cg < CG; ++cg) {
                c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[cg], b[gi][cg], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[cg], b[gi][cg], c1, 0, 0, 0);
            }
            const int a8[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
            const v2i r = epi8_quant_i8p8<EPI == EPI_I8_P8_NONNEG>(ep, prm, a8);
            const int pix = pix0 + 16 * gi + p;
            const unsigned oo = (orow + pix) * 8u;
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, r), rout, (int)(live && pix < HW ? oo : PW_OOB),
                                                  0, 0);
        }
    }
}

// The upper clamp of the rounded result per channel for the ReLU / clip epilogue, as epi8_clamp_pair packs it: two
// 16-bit values per dword. Host arithmetic in the order the kernels use (one multiplication, one addition, toward zero).
void conv_pw_stream_clamps(float act_hi, float round_half, const float* scale_out, int n, unsigned* dst) {
    auto one = [&](float so) {
        float t = act_hi * so;
        t = t + round_half;
        return t >= 127.f ? 127u : (unsigned)(int)t;
    };
    for (int i = 0; i + 1 < n; i += 2) dst[i / 2] = one(scale_out[i]) | one(scale_out[i + 1]) << 16;
}

bool conv_pw_stream_applicable(const ConvGeom& g, const Epilogue& ep) {
    if (g.groups != 1 || g.kh != 1 || g.kw != 1 || g.sh != 1 || g.sw != 1 || g.ph != 0 || g.pw != 0) return false;
    if (g.Cs || g.Ks || g.C % 8 || g.C > 64 * PW_MAX_CG || g.K % 8 || g.N < 1 || g.N > 65535) return false;
    if ((size_t)std::max(g.C, g.K) * g.H * g.W >= (1ull << 31)) return false;  // 32-bit offsets inside an image
    // More than one reduction step: a workgroup copies 2 KB of weights per step and channel pair into LDS for its 128
    // pixels, which pays on large blobs with four steps. Measured against the implicit-GEMM kernel (kernel trace of the
    // layer alone, us): 256 -> 512 @28x28 b32 12.8 / 14.0, 256 -> 64 @56x56 b16 6.1 / 7.3. With two or three steps the
    // kernel also ran 128 -> 128 @28x28 b64 at 7.0 / 8.4, but 176 -> 176 @26x26 b16 at 5.9 / 5.0, and the pointwise
    // layers of the two benchmark networks that would take it (88 .. 176 channels) made their passes 0.3 - 1 % slower on
    // the same box (cold inputs): those stay on the implicit-GEMM kernel.
    if (g.C > 64 && (g.C <= 192 || (long)g.N * g.H * g.W < 20000)) return false;
    const int epi = pick_epilogue(ep, g.K);
    return epi == EPI_I8_P8 || epi == EPI_I8_P8_NONNEG;
}

// Pixel groups per wave and slices of the channel pairs. Four groups per wave amortize a pair's operand reads best
// and are taken while they still leave every SIMD a few waves; below that two groups, and the channel pairs cut
// into slices (each slice re-reads the pixels, which are few bytes next to what it writes) until there are about
// two waves per SIMD or a slice is down to two pairs.
void conv_pw_stream_plan(const ConvGeom& g, int* groups, int* slices) {
    const int HW = g.H * g.W, pairs = (g.K + 31) / 32;
    auto waves = [&](int G, int s) { return (long)g.N * ((HW + 16 * G - 1) / (16 * G)) * s; };
    const int G = waves(4, 1) >= 8192 ? 4 : 2;
    int s = 1;
    const int smax = std::max(1, pairs / 2);
    while (s < smax && waves(G, s) < 8192) ++s;
    while ((pairs + s - 1) / s > pw_max_pairs((g.C + 63) / 64)) ++s;  // a slice's LDS image stays under 64 KB
    const int per = (pairs + s - 1) / s;
    *groups = G, *slices = (pairs + per - 1) / per;
}

template <int EPI, int G, int CG>
static hipError_t launch_pw(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                            const unsigned* qh, int slices, hipStream_t stream) {
    const int HW = g.H * g.W, pairs = (g.K + 31) / 32;
    const int per = (pairs + slices - 1) / slices;
    const dim3 grid((HW + 64 * G - 1) / (64 * G), g.N, (pairs + per - 1) / per);
    hipLaunchKernelGGL((conv_pw_stream_kernel<EPI, G, CG>), grid, dim3(256), (size_t)per * pw_pair_v4(CG) * 16, stream, x, wpk,
                       (int8_t*)out, ep, qh, g.C / 8, g.K, HW, per, igemm_padded_rows(g.K) / 16);
    return hipGetLastError();
}

// qh: conv_pw_stream_clamps of the layer's output scales (read by the ReLU / clip epilogue only)
// force_groups / force_slices: 0 = automatic
hipError_t run_conv_pw_stream(const int8_t* x, const int8_t* wpk, const unsigned* qh, void* out, const ConvGeom& g,
                              const Epilogue& ep, int force_groups, int force_slices, hipStream_t stream) {
    if (!conv_pw_stream_applicable(g, ep)) return hipErrorInvalidValue;
    int G, s;
    conv_pw_stream_plan(g, &G, &s);
    if (force_groups) G = force_groups;
    if (force_slices) s = force_slices;
    const int pairs = (g.K + 31) / 32, cgs = (g.C + 63) / 64;
    if ((G != 2 && G != 4) || s < 1 || s > pairs) return hipErrorInvalidValue;
    if (cgs > 1) G = 2;  // (four groups of four reduction steps are more operand registers than pay)
    while ((pairs + s - 1) / s > pw_max_pairs(cgs)) ++s;  // a slice's LDS image stays under 64 KB
    const bool nonneg = pick_epilogue(ep, g.K) == EPI_I8_P8_NONNEG;
    if (nonneg && !qh) return hipErrorInvalidValue;
#define OHIP_PW(G_, CG_) \
    if (G == G_ && cgs == CG_) \
        return nonneg ? launch_pw<EPI_I8_P8_NONNEG, G_, CG_>(x, wpk, out, g, ep, qh, s, stream) \
                      : launch_pw<EPI_I8_P8, G_, CG_>(x, wpk, out, g, ep, qh, s, stream);
    OHIP_PW(4, 1)
    OHIP_PW(2, 1)
    OHIP_PW(2, 4)
#undef OHIP_PW
    return hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------------------------------------------
// A pointwise int8 convolution with an fp32 result whose only reader is the mean over the image (the tail of a
// classifier: head convolution, global average pooling): out[n][k] = mean over H*W of activation(acc * scale_in + bias),
// one launch, the convolution's own blob (H*W times the size of the result) never written or read back.
// A wave owns a pair of 16-row tiles (32 output channels, igemm_row_channel) x all pixels of one image (at most 64: four
// groups of 16 as the B operands of every reduction step, loaded straight from the Byte8 blob; the four waves of a
// workgroup read the same pixels, which the first one brings into the CU's cache). After the last step a lane holds,
// per tile, four channels of its pixel in each group: it adds the activated values of its groups, the 16 lanes of a
// row group add theirs (xor butterfly), and lane 0 of the group stores four means.
template <int CGS>  // reduction steps of 64 input channels when they are at most 5 (all operands requested at once); 0: a loop
__global__ void __launch_bounds__(256) conv_pw_avgpool_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk,
                                                              float* __restrict__ out, ConvGeom g, Epilogue ep, int cgs,
                                                              int mt16) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
    const int pair = blockIdx.x * 4 + wave, img = blockIdx.y;
    if (2 * pair >= mt16) return;  // whole wave
    const int HW = g.H * g.W, C8 = g.C / 8;
    v4i acc[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int p = 0; p < 4; ++p) acc[t][p] = v4i{0, 0, 0, 0};
    const v4i* wv = reinterpret_cast<const v4i*>(wpk);
    // (every load is unconditional: a pixel or an octet that does not exist carries an offset past the buffer and reads
    // zero; behind per-lane branches the compiler would wait for each load before it issues the next)
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(x), 0, (int)((size_t)g.N * g.C * HW), 0x00020000);
    const unsigned s_img = (unsigned)img * (unsigned)(C8 * HW) * 8u;
    const int second = 2 * pair + 1 < mt16 ? 1 : 0;  // (an odd tile count: the pair's second tile repeats the first, unused)
    auto load = [&](int cg, v4i (&a)[2], v4i (&b)[4]) {
        a[0] = wv[((size_t)cg * mt16 + 2 * pair) * 64 + lane];
        a[1] = wv[((size_t)cg * mt16 + 2 * pair + second) * 64 + lane];
        const int oct = cg * 8 + 2 * q;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int pix = 16 * p + n;
            const unsigned v0 = (pix < HW && oct < C8) ? (unsigned)(oct * HW + pix) * 8u : PW_OOB;
            const unsigned v1 = (pix < HW && oct + 1 < C8) ? (unsigned)((oct + 1) * HW + pix) * 8u : PW_OOB;
            const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rx, (int)v0, (int)s_img, 0));
            const v2i hi = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rx, (int)v1, (int)s_img, 0));
            b[p] = v4i{lo[0], lo[1], hi[0], hi[1]};
        }
    };
    auto mac = [&](const v4i (&a)[2], const v4i (&b)[4]) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            acc[0][p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], b[p], acc[0][p], 0, 0, 0);
            acc[1][p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[1], b[p], acc[1][p], 0, 0, 0);
        }
    };
    if constexpr (CGS > 0) {
        v4i a[CGS][2], b[CGS][4];
#pragma unroll
        for (int cg = 0; cg < CGS; ++cg) load(cg, a[cg], b[cg]);
#pragma unroll
        for (int cg = 0; cg < CGS; ++cg) mac(a[cg], b[cg]);
    } else {
        v4i a[2][2], b[2][4];
        load(0, a[0], b[0]);
        for (int cg = 0; cg < cgs; cg += 2) {  // the next step's operands are requested before this step's are used
            load(min(cg + 1, cgs - 1), a[1], b[1]);
            mac(a[0], b[0]);
            if (cg + 1 < cgs) {
                load(min(cg + 2, cgs - 1), a[0], b[0]);
                mac(a[1], b[1]);
            }
        }
    }
    const float count = (float)HW;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int ch0 = 32 * pair + 8 * q + 4 * t;  // igemm_row_channel of rows 4q .. 4q+3 of tile 2 pair + t
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ch = ch0 + e;
            const bool live = ch < g.K;
            const float si = ep.scale_in[ch], bi = ep.bias[ch];  // (the arrays are padded to whole row blocks)
            float s = 0.f;
#pragma unroll
            for (int p = 0; p < 4; ++p)
                if (16 * p + n < HW) s += activate(__fmaf_rn((float)acc[t][p][e], si, bi), ep.act, ep.act_p0);
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) s += __shfl_xor(s, o, 16);
            if (n == 0 && live) out[(size_t)img * g.K + ch] = s / count;
        }
    }
}

bool conv_pw_avgpool_applicable(const ConvGeom& g, const Epilogue& ep) {
    if (g.kh != 1 || g.kw != 1 || g.sh != 1 || g.sw != 1 || g.ph || g.pw || g.groups != 1 || g.C % 8) return false;
    if (ep.out_kind != OTTER_HIP_OUT_F32 || ep.twin || ep.residual) return false;
    if ((size_t)g.N * g.C * g.H * g.W >= ((size_t)1 << 31)) return false;
    return g.H * g.W <= 64 && g.N <= 65535;
}

hipError_t run_conv_pw_avgpool(const int8_t* x, const int8_t* wpk, float* out, const ConvGeom& g, const Epilogue& ep,
                               hipStream_t stream) {
    if (g.N == 0) return hipSuccess;
    const int mt16 = igemm_padded_rows(g.K) / 16, pairs = (mt16 + 1) / 2;
    const int cgs = igemm_channel_groups(g.C);
    const dim3 grid((unsigned)((pairs + 3) / 4), (unsigned)g.N);
#define OHIP_PWA(N_) hipLaunchKernelGGL(conv_pw_avgpool_kernel<N_>, grid, dim3(256), 0, stream, x, wpk, out, g, ep, cgs, mt16)
    switch (cgs) {
    case 1: OHIP_PWA(1); break;
    case 2: OHIP_PWA(2); break;
    case 3: OHIP_PWA(3); break;
    case 4: OHIP_PWA(4); break;
    case 5: OHIP_PWA(5); break;
    default: OHIP_PWA(0); break;
    }
#undef OHIP_PWA
    return hipGetLastError();
}

}  // namespace ohip
