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
typedef unsigned v4u_store __attribute__((__vector_size__(4 * sizeof(unsigned))));

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
// The pointwise layer on an fp32 Float8 blob (quantize_to_int8 of Tensor/ConvolutionLayer.cpp:770-775 and the convolution
// as one launch), int8 or fp32 result, up to 256 input channels.
//
// The blob is four times the bytes of its int8 copy, so it is read ONCE: a wave owns G groups of 16 pixels of one image,
// requests all their channels at the start of the kernel (4 x 16 bytes per lane, group and reduction step: the bytes in
// flight per wave are what keeps HBM busy on a layer of a few thousand waves), quantizes them into the B operands it
// keeps for the whole kernel, and walks ALL output channels in pairs of 16-row tiles. The pairs' weights and constants
// go through LDS in rounds of `pairs_per_round` (the image of conv_pw_stream_kernel; a barrier on either side of a
// round's copy), so a round's LDS stays small enough for several workgroups per compute unit.
// fp32 result (EPI_F32_P4): after the MFMAs of a pair a lane holds two Float4 elements of its pixel (igemm_row_channel).
constexpr int PW_F32IN_COPIES = 9;  // 16-byte loads per thread and round of the weight image

template <int EPI, int G, int CG>
__global__ void __launch_bounds__(256) conv_pw_f32in_kernel(const float* __restrict__ x, const int8_t* __restrict__ wpk,
                                                            void* __restrict__ out, Epilogue ep,
                                                            const unsigned* __restrict__ qh, int C8, int K, int HW,
                                                            int pairs_per_round, int mt, const float* __restrict__ in_scale_p,
                                                            float in_half) {
    constexpr int PW_PAIR_V4 = pw_pair_v4(CG);
    constexpr bool F32 = EPI == EPI_F32_P4;
    constexpr int W4 = 128 * CG;
    extern __shared__ v4i pw_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane >> 4, p = lane & 15;
    const int n = blockIdx.y;
    const int pix0 = (blockIdx.x * 4 + wave) * (16 * G);
    const bool active = pix0 < HW;  // (a wave past the image still copies and meets the barriers)

    const size_t in_img = (size_t)C8 * HW * 32, out_img = (size_t)K * HW * (F32 ? 4 : 1);
    const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(x)) + (size_t)n * in_img, 0, (int)in_img, 0x00020000);
    const __amdgpu_buffer_rsrc_t rout =
        __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(out) + (size_t)n * out_img, 0, (int)out_img, 0x00020000);

    // every byte the wave will read, requested now (pixels or octets that do not exist: past the buffer, zeros)
    v4i raw[G][CG][4];
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
        const int pix = pix0 + 16 * gi + p;
        const bool in = pix < HW;
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            const int oct = 8 * cg + 2 * q;
            const unsigned o0 = ((unsigned)oct * HW + pix) * 32u;
            const int v0 = (int)(in && oct < C8 ? o0 : PW_OOB), v1 = (int)(in && oct + 1 < C8 ? o0 + (unsigned)HW * 32u : PW_OOB);
            raw[gi][cg][0] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, v0, 0, 0));
            raw[gi][cg][1] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, v0 + 16, 0, 0));
            raw[gi][cg][2] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, v1, 0, 0));
            raw[gi][cg][3] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, v1 + 16, 0, 0));
        }
    }
    const float in_scale = in_scale_p[0];
    // float2int8 of four values into four bytes (the arithmetic of otter_hip_quantize)
    auto quant4 = [&](const v4i& f) -> int {
        int k[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float t = __fmul_rn(__int_as_float(f[e]), in_scale);
            k[e] = (int)__fadd_rn(t, __builtin_copysignf(in_half, t));  // toward zero, saturating
        }
        const ohip_v2s top = {127, 127}, bot = {-127, -127};
        ohip_v2s a = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(k[0], k[1]));
        ohip_v2s b = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(k[2], k[3]));
        a = __builtin_elementwise_max(__builtin_elementwise_min(a, top), bot);
        b = __builtin_elementwise_max(__builtin_elementwise_min(b, top), bot);
        return (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, b), __builtin_bit_cast(unsigned, a), 0x06040200u);
    };
    v4i b[G][CG];

    const int pairs = (K + 31) / 32;
    const v4i* wg = reinterpret_cast<const v4i*>(wpk);
    const v4i* sg = reinterpret_cast<const v4i*>(ep.scale_in);
    const v4i* bg = reinterpret_cast<const v4i*>(ep.bias);
    const v4i* og = reinterpret_cast<const v4i*>(ep.scale_out);
    const v4i* cq = reinterpret_cast<const v4i*>(qh);
    // A round's image, copied by all threads with PW_F32IN_COPIES loads each: slot k of a thread is element
    // threadIdx.x + 256 k of the image, i.e. always the same array and the same place in a pair, one round further each
    // time (a pointer and its step per slot). The loads are unconditional (a slot past the image or past the last pair
    // reads the first weights again and lands in the slack of the buffer) and are requested before the round in front
    // is computed; the image goes into the other of two LDS buffers once that is done: one barrier per round.
    // The per-channel arrays are padded to the weight rows, so every pair is whole in memory.
    constexpr int BUF_V4 = 256 * PW_F32IN_COPIES;
    const v4i* src[PW_F32IN_COPIES];
    int step[PW_F32IN_COPIES], prk[PW_F32IN_COPIES];
#pragma unroll
    for (int k = 0; k < PW_F32IN_COPIES; ++k) {
        const int i = threadIdx.x + 256 * k;
        const int pr = i / PW_PAIR_V4, r = i % PW_PAIR_V4;
        src[k] = wg + ((size_t)(r / 128) * mt + 2 * pr) * 64 + r % 128;  // (step, the pair's two tiles, lane)
        step[k] = 2 * pairs_per_round * 64;
        if (r >= W4) src[k] = sg + pr * 8 + r - W4, step[k] = pairs_per_round * 8;
        if (r >= W4 + 8) src[k] = bg + pr * 8 + r - W4 - 8;
        if (r >= W4 + 16) {
            if constexpr (F32) src[k] = wg, step[k] = 0;
            else src[k] = og + pr * 8 + r - W4 - 16;
        }
        if (r >= W4 + 24) {
            if constexpr (EPI == EPI_I8_P8_NONNEG) src[k] = cq + pr * 4 + r - W4 - 24, step[k] = pairs_per_round * 4;
            else src[k] = wg, step[k] = 0;
        }
        prk[k] = pr;
        if (pr >= pairs_per_round) src[k] = wg, step[k] = 0, prk[k] = 0;
    }
    v4i cp[PW_F32IN_COPIES];
    auto copy_request = [&](int pr0) {
#pragma unroll
        for (int k = 0; k < PW_F32IN_COPIES; ++k) {
            cp[k] = *(pr0 + prk[k] < pairs ? src[k] : wg);
            src[k] += step[k];
        }
    };
    auto copy_store = [&](int buf) {
#pragma unroll
        for (int k = 0; k < PW_F32IN_COPIES; ++k) pw_lds[buf * BUF_V4 + threadIdx.x + 256 * k] = cp[k];
    };
    // A pair in two steps: its products (the A operands from LDS, two chains of CG matrix instructions per group) and
    // its epilogue (constants from LDS, dequantize or requantize, stores). (Issuing the next pair's products in front of
    // the current epilogue changed nothing measurable: the rounds wait for the stores, not for the matrix pipe.)
    auto products = [&](const v4i* l, v4i (&c0)[G], v4i (&c1)[G]) {
        v4i a0[CG], a1[CG];
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) a0[cg] = l[128 * cg + lane], a1[cg] = l[128 * cg + 64 + lane];
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
            c0[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[0], b[gi][0], v4i{0, 0, 0, 0}, 0, 0, 0);
            c1[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[0], b[gi][0], v4i{0, 0, 0, 0}, 0, 0, 0);
        }
#pragma unroll
        for (int cg = 1; cg < CG; ++cg)
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
                c0[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[cg], b[gi][cg], c0[gi], 0, 0, 0);
                c1[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[cg], b[gi][cg], c1[gi], 0, 0, 0);
            }
    };
    auto epilogue = [&](const v4i* l, int pr, const v4i (&c0)[G], const v4i (&c1)[G]) {
        const v4i s0 = l[W4 + 2 * q], s1 = l[W4 + 1 + 2 * q], b0 = l[W4 + 8 + 2 * q], b1 = l[W4 + 9 + 2 * q];
        const int ch0 = 32 * pr + 8 * q;
        if constexpr (F32) {
            float si[8], bi[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                si[e] = __int_as_float(s0[e]), si[4 + e] = __int_as_float(s1[e]);
                bi[e] = __int_as_float(b0[e]), bi[4 + e] = __int_as_float(b1[e]);
            }
            const unsigned orow = (unsigned)(ch0 >> 2) * HW;
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
                const int pix = pix0 + 16 * gi + p;
                const v4i r0 = ep.lrelu ? epi4_dequant_f32p4<true>(ep, si, bi, c0[gi][0], c0[gi][1], c0[gi][2], c0[gi][3])
                                        : epi4_dequant_f32p4<false>(ep, si, bi, c0[gi][0], c0[gi][1], c0[gi][2], c0[gi][3]);
                const v4i r1 = ep.lrelu ? epi4_dequant_f32p4<true>(ep, si + 4, bi + 4, c1[gi][0], c1[gi][1], c1[gi][2], c1[gi][3])
                                        : epi4_dequant_f32p4<false>(ep, si + 4, bi + 4, c1[gi][0], c1[gi][1], c1[gi][2], c1[gi][3]);
                const unsigned oo = (orow + pix) * 16u;
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_store, r0), rout,
                                                       (int)(ch0 < K && pix < HW ? oo : PW_OOB), 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_store, r1), rout,
                                                       (int)(ch0 + 4 < K && pix < HW ? oo + (unsigned)HW * 16u : PW_OOB), 0, 0);
            }
        } else {
            Epi8 prm;
            const v4i o0 = l[W4 + 16 + 2 * q], o1 = l[W4 + 17 + 2 * q], c = l[W4 + 24 + q];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                prm.si[e] = __int_as_float(s0[e]), prm.si[4 + e] = __int_as_float(s1[e]);
                prm.bi[e] = __int_as_float(b0[e]), prm.bi[4 + e] = __int_as_float(b1[e]);
                prm.so[e] = __int_as_float(o0[e]), prm.so[4 + e] = __int_as_float(o1[e]);
                prm.qh[e] = (unsigned)c[e];
            }
            const bool live = ch0 < K;
            const unsigned orow = (unsigned)(ch0 >> 3) * HW;
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
                const int a8[8] = {c0[gi][0], c0[gi][1], c0[gi][2], c0[gi][3], c1[gi][0], c1[gi][1], c1[gi][2], c1[gi][3]};
                const v2i r = epi8_quant_i8p8<EPI == EPI_I8_P8_NONNEG>(ep, prm, a8);
                const int pix = pix0 + 16 * gi + p;
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, r), rout,
                                                      (int)(live && pix < HW ? (orow + pix) * 8u : PW_OOB), 0, 0);
            }
        }
    };
    auto compute = [&](int pr0, int pr1, int buf) {
        const v4i* l = pw_lds + buf * BUF_V4;
        for (int pr = pr0; pr < pr1; ++pr, l += PW_PAIR_V4) {
            v4i c0[G], c1[G];
            products(l, c0, c1);
            epilogue(l, pr, c0, c1);
        }
    };

    copy_request(0);
    __builtin_amdgcn_sched_barrier(0);  // (everything in flight before anything waits for the first)
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
            b[gi][cg] = v4i{quant4(raw[gi][cg][0]), quant4(raw[gi][cg][1]), quant4(raw[gi][cg][2]), quant4(raw[gi][cg][3])};
    copy_store(0);
    __syncthreads();
    for (int pr0 = 0, buf = 0; pr0 < pairs; pr0 += pairs_per_round, buf ^= 1) {
        const bool more = pr0 + pairs_per_round < pairs;
        if (more) copy_request(pr0 + pairs_per_round);
        if (active) compute(pr0, min(pr0 + pairs_per_round, pairs), buf);
        if (more) copy_store(buf ^ 1);  // (last read before the barrier that ended the round in front)
        __syncthreads();
    }
}

// a round is what the 256 threads copy with PW_F32IN_COPIES loads each (36 KB: four workgroups fit a compute unit)
static int pw_f32in_pairs_per_round(int cgs, int pairs) { return std::max(1, std::min(pairs, 256 * PW_F32IN_COPIES / pw_pair_v4(cgs))); }

bool conv_pw_f32in_applicable(const ConvGeom& g, const Epilogue& ep) {
    if (g.groups != 1 || g.kh != 1 || g.kw != 1 || g.sh != 1 || g.sw != 1 || g.ph != 0 || g.pw != 0) return false;
    if (g.Cs || g.Ks || g.C % 8 || g.C > 64 * PW_MAX_CG || g.N < 1 || g.N > 65535) return false;
    if (ep.twin != nullptr || ep.residual != nullptr) return false;
    const int epi = pick_epilogue(ep, g.K);
    if (epi != EPI_I8_P8 && epi != EPI_I8_P8_NONNEG && epi != EPI_F32_P4) return false;
    if (g.K % (epi == EPI_F32_P4 ? 4 : 8)) return false;
    // 32-bit byte offsets inside an image of either blob
    return (size_t)g.C * g.H * g.W * 4 < (1ull << 31) && (size_t)g.K * g.H * g.W * 4 < (1ull << 31);
}

template <int EPI, int G, int CG>
static hipError_t launch_pw_f32in(const float* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                  const unsigned* qh, int per, const float* in_scale, float in_half, hipStream_t stream) {
    auto kern = conv_pw_f32in_kernel<EPI, G, CG>;
    constexpr size_t lds = (size_t)2 * 256 * PW_F32IN_COPIES * 16;  // two buffers of a round's image
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int HW = g.H * g.W;
    const dim3 grid((HW + 64 * G - 1) / (64 * G), g.N, 1);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, x, wpk, out, ep, qh, g.C / 8, g.K, HW, per,
                       igemm_padded_rows(g.K) / 16, in_scale, in_half);
    return hipGetLastError();
}

// qh: conv_pw_stream_clamps of the layer's output scales (read by the ReLU / clip epilogue only)
// force_groups / force_pairs: 0 = automatic
hipError_t run_conv_pw_f32in(const float* x, const int8_t* wpk, const unsigned* qh, void* out, const ConvGeom& g, const Epilogue& ep,
                             const float* in_scale, int in_round_mode, int force_groups, int force_pairs, hipStream_t stream) {
    if (!conv_pw_f32in_applicable(g, ep)) return hipErrorInvalidValue;
    const int HW = g.H * g.W, pairs = (g.K + 31) / 32, cgs = (g.C + 63) / 64;
    // two groups per wave halve the LDS reads per output; one group while two would leave SIMDs without a wave
    int G = (long)g.N * ((HW + 31) / 32) >= 1024 ? 2 : 1;
    if (force_groups) G = force_groups;
    if (G != 1 && G != 2) return hipErrorInvalidValue;
    int per = pw_f32in_pairs_per_round(cgs, pairs);
    if (force_pairs) per = std::min(std::min(force_pairs, per), pairs);
    const int epi = pick_epilogue(ep, g.K);
    if (epi == EPI_I8_P8_NONNEG && !qh) return hipErrorInvalidValue;
    const float half = in_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
#define OHIP_PWF(E_, G_, CG_) \
    if (epi == E_ && G == G_ && cgs == CG_) return launch_pw_f32in<E_, G_, CG_>(x, wpk, out, g, ep, qh, per, in_scale, half, stream);
#define OHIP_PWF_E(G_, CG_) OHIP_PWF(EPI_I8_P8, G_, CG_) OHIP_PWF(EPI_I8_P8_NONNEG, G_, CG_) OHIP_PWF(EPI_F32_P4, G_, CG_)
    OHIP_PWF_E(1, 1) OHIP_PWF_E(1, 2) OHIP_PWF_E(1, 3) OHIP_PWF_E(1, 4)
    OHIP_PWF_E(2, 1) OHIP_PWF_E(2, 2) OHIP_PWF_E(2, 3) OHIP_PWF_E(2, 4)
#undef OHIP_PWF_E
#undef OHIP_PWF
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
