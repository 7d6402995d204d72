// Dense int8 convolution as an implicit GEMM on the gfx950 matrix cores (v_mfma_i32_16x16x64_i8).
//
//   D[M = out channel][N = pixel] = sum_k  Wp[M][k] * X[k][N],   k = (tap, input channel)
//
// Activations stay in the reference's Byte8 layout [N, C/8, H, W, 8] (no im2col, no padded copy): a k-chunk
// of 64 is one filter tap x 64 input channels = 8 channel octets of one input pixel, and a lane's 16-byte
// MFMA operand is two neighbouring octets. Out-of-image taps are predicated to zero.
// Weights are re-laid-out once on the host into the exact lane order the MFMA consumes
// ([k-chunk][16-row tile][lane][16 B]), so the global->LDS copy and the LDS->register reads are linear.
// Output rows are permuted (see igemm_row_channel) so that after the MFMA each lane owns 8 consecutive output
// channels of one pixel: one 8-byte Byte8 store, or two 16-byte Float4 / Int4 stores, per lane, with the 16
// lanes of a row group covering 16 consecutive pixels -- the reference's packed layouts come out directly.
#include "common.hpp"
#include "conv_igemm.hpp"

#include <algorithm>
#include <type_traits>

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

template <int TM, int TN, int WM, int WN>
struct IgemmCfg {
    static constexpr int kThreads = 256;
    static constexpr int FM = TM / WM / 16;          // 16-row fragments per wave
    static constexpr int FN = TN / WN / 16;          // 16-pixel fragments per wave
    static constexpr int A_BYTES = TM * 64;          // weights per k-chunk
    static constexpr int B_BYTES = TN * 64;          // activations per k-chunk
    static constexpr int A_V = (A_BYTES / 16 + kThreads - 1) / kThreads;  // 16-byte vectors per thread
    static constexpr int B_V = TN / 64;                                   // (pixel, octet pair) items per thread
    static_assert(WM * WN == 4, "four waves");
    static_assert(FM >= 2 && FM % 2 == 0, "row fragments come in pairs");
    static_assert(TN % 64 == 0, "pixel tile");
};

// KC = k-chunks per stage. KC == 1: LDS double buffer, the next chunk in registers while one is multiplied (one
// global-memory latency per chunk: right for long reductions, where several workgroups per CU cover it). KC > 1: a
// stage of KC chunks in a single LDS buffer, the whole next stage in registers meanwhile; a reduction of at most KC
// chunks (pointwise layers) then pays the latency once per workgroup instead of once per chunk.
// INF: the input is the fp32 Float8 blob of a pointwise layer ([N][C/8][H*W][8 floats]); the loader reads the 32 bytes
// of a pixel's octet and quantizes them with the layer's input scale and rounding primitive on the way into LDS
// (quantize_to_int8, Tensor/ConvolutionLayer.cpp:770-775, without its own pass over the blob).
template <int TM, int TN, int WM, int WN, int EPI, int KC, bool INF = false>
__global__ void __launch_bounds__(256) conv_igemm_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk,
                                                         void* __restrict__ out, ConvGeom g, Epilogue ep, int m_tiles16,
                                                         int c_groups, int n_pix_tiles, const float* __restrict__ in_scale_p,
                                                         float in_half) {
    using Cfg = IgemmCfg<TM, TN, WM, WN>;
    constexpr int FM = Cfg::FM, FN = Cfg::FN;
    constexpr int NBUF = KC == 1 ? 2 : KC;
    __shared__ __attribute__((aligned(16))) int8_t lds_a[NBUF][Cfg::A_BYTES];
    __shared__ __attribute__((aligned(16))) int8_t lds_b[NBUF][Cfg::B_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    // Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous run of pixel tiles so
    // that neighbouring tiles (which share halo rows and all weights) meet in the same L2.
    int pt = blockIdx.x;
    {
        const int per = n_pix_tiles / 8;
        if (per > 0 && pt < per * 8) pt = (pt % 8) * per + pt / 8;
    }
    const int mt0 = blockIdx.y * (TM / 16);  // first 16-row tile of this workgroup
    const int OHW = g.OH * g.OW;
    // Grouped convolution: blockIdx.z is the group, g.C / g.K are ONE group's channels and g.Cs / g.Ks the tensors'.
    // A group is a channel slice of both tensors (whole octets in, whole output elements out), with its own block of
    // packed weights and its own run of the per-channel constants.
    const int Cs8 = (g.Cs ? g.Cs : g.C) / 8;
    const int Ks = g.Ks ? g.Ks : g.K;
    if (blockIdx.z) {
        const int grp = blockIdx.z;
        x += (size_t)grp * (g.C / 8) * g.H * g.W * 8;
        wpk += (size_t)grp * (g.tap_pack > 1 ? (g.kh * g.kw + g.tap_pack - 1) / g.tap_pack : g.kh * g.kw * c_groups) * m_tiles16 * 1024;
        out = (char*)out + (size_t)grp * g.K * OHW * (EPI == EPI_I8_P8 || EPI == EPI_I8_P8_NONNEG ? 1 : 4);
        ep.scale_in += grp * g.K;
        ep.bias += grp * g.K;
        if (ep.scale_out) ep.scale_out += grp * g.K;
    }
    // 32-bit pixel indices: the C ABI refuses tensors of 2^31 elements or more, and a 64-bit division costs ~4x
    const unsigned total_pix = (unsigned)g.N * (unsigned)OHW;
    const unsigned tile_base = (unsigned)pt * TN;
    const int C8 = g.C / 8;
    const int HW = g.H * g.W;

    // ---- per-thread constants of the activation loader -------------------------------------------
    // (image, pixel) of a global pixel index: the tile's first pixel is divided once for the whole workgroup (uniform
    // operands), a lane then only steps over at most one image boundary; images smaller than a tile take the division
    const unsigned n_tile = tile_base / (unsigned)OHW;
    const unsigned rem_tile = tile_base - n_tile * (unsigned)OHW;
    auto locate = [&](unsigned ofs, unsigned& n, unsigned& pix) {  // pixel tile_base + ofs, ofs < TN
        n = n_tile, pix = rem_tile + ofs;
        if ((unsigned)OHW >= (unsigned)TN) {
            if (pix >= (unsigned)OHW) pix -= (unsigned)OHW, ++n;
        } else {
            const unsigned k = pix / (unsigned)OHW;
            n += k, pix -= k * (unsigned)OHW;
        }
    };
    // a pointwise layer (1x1, stride 1, no padding) reads input pixel = output pixel: no row / column split, no bounds
    const bool pointwise = g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0;
    const int p_l = tid % TN;
    const int j0 = tid / TN;
    constexpr int J_STEP = 256 / TN > 0 ? 256 / TN : 1;
    const bool pvalid = tile_base + p_l < total_pix;
    int iy0 = 0, ix0 = 0;
    // this thread's pixel at tap (0, 0), octet 0, as a byte offset into the (group's slice of the) input; the loads go
    // through a buffer descriptor, so that an out-of-image tap or a padded octet is an out-of-range offset (reads as
    // zero) instead of a branch around the load
    int px_ofs = 0;
    if (pvalid) {
        unsigned n, pix;
        locate((unsigned)p_l, n, pix);
        const int img = (int)n * Cs8 * HW * 8;
        if (pointwise) {
            px_ofs = img + (int)pix * 8;
        } else {
            const int oy = (int)(pix / (unsigned)g.OW), ox = (int)pix - oy * g.OW;
            iy0 = oy * g.sh - g.ph;
            ix0 = ox * g.sw - g.pw;
            px_ofs = img + (iy0 * g.W + ix0) * 8;
        }
    }
    constexpr unsigned IG_OOB = 0x80000000u;
    const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(x), 0,
        (int)(((unsigned)g.N * (unsigned)Cs8 * (unsigned)HW * 8u - (unsigned)blockIdx.z * (unsigned)(g.C / 8) * (unsigned)HW * 8u) * (INF ? 4u : 1u)),
        0x00020000);

    v2i breg[INF ? 1 : KC][INF ? 1 : Cfg::B_V][2];
    v4i bregf[INF ? KC : 1][INF ? Cfg::B_V : 1][4];  // INF: two octets x 8 floats of a pixel
    float in_scale = 0.f;
    if constexpr (INF) in_scale = in_scale_p[0];
    v4i areg[KC][Cfg::A_V];
    // Few input channels (a group of a grouped convolution with at most 32): tap_pack kernel taps share a reduction
    // step, the 16-channel quarter j of the step being channels 16 (j % per) .. of tap tap_pack * kc + j / per with
    // per = 4 / tap_pack quarters per tap (j is the same for a whole wave: a pixel tile is at least 64 wide)
    const int tpk = g.tap_pack > 1 ? g.tap_pack : 1;
    const int n_chunks = tpk > 1 ? (g.kh * g.kw + tpk - 1) / tpk : g.kh * g.kw * c_groups;

    auto load_global = [&](int kc, int q) {
        if (tpk > 1) {  // (uniform)
            const int per = 4 / tpk;
#pragma unroll
            for (int r = 0; r < Cfg::B_V; ++r) {
                const int j = j0 + r * J_STEP;
                const int tap = kc * tpk + j / per;
                const int u = tap / g.kw, v = tap - u * g.kw;
                const int iy = iy0 + u * g.dh, ix = ix0 + v * g.dw;
                const bool inb = pvalid && tap < g.kh * g.kw && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                const int o0 = 2 * (j % per);
                const unsigned v_lo = (unsigned)(px_ofs + ((u * g.dh) * g.W + v * g.dw) * 8 + o0 * HW * 8);
                breg[q][r][0] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(inb && o0 < C8 ? v_lo : IG_OOB), 0, 0));
                breg[q][r][1] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(
                    rin, (int)(inb && o0 + 1 < C8 ? v_lo + (unsigned)(HW * 8) : IG_OOB), 0, 0));
            }
        } else {
        const int tap = kc / c_groups, cgp = kc % c_groups;
        const int u = tap / g.kw, v = tap % g.kw;
        bool inb = pvalid;
        if (!pointwise) {
            const int iy = iy0 + u * g.dh, ix = ix0 + v * g.dw;
            inb = pvalid && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
        }
        const int tap_ofs = ((u * g.dh) * g.W + v * g.dw) * 8;  // (uniform)
#pragma unroll
        for (int r = 0; r < Cfg::B_V; ++r) {
            const int o0 = cgp * 8 + 2 * (j0 + r * J_STEP);
            const unsigned v_lo = (unsigned)(px_ofs + tap_ofs + o0 * HW * 8);
            if constexpr (INF) {
                // (the fp32 element of a pixel's octet lies at four times the int8 element's offset)
                const unsigned f0 = inb && o0 < C8 ? v_lo * 4u : IG_OOB, f1 = inb && o0 + 1 < C8 ? (v_lo + (unsigned)(HW * 8)) * 4u : IG_OOB;
                bregf[q][r][0] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)f0, 0, 0));
                bregf[q][r][1] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)f0, 16, 0));
                bregf[q][r][2] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)f1, 0, 0));
                bregf[q][r][3] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)f1, 16, 0));
            } else {
                breg[q][r][0] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(inb && o0 < C8 ? v_lo : IG_OOB), 0, 0));
                breg[q][r][1] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(
                    rin, (int)(inb && o0 + 1 < C8 ? v_lo + (unsigned)(HW * 8) : IG_OOB), 0, 0));
            }
        }
        }
        const int8_t* wa = wpk + ((size_t)kc * m_tiles16 + mt0) * 1024;
#pragma unroll
        for (int r = 0; r < Cfg::A_V; ++r) {
            const int vi = tid + r * 256;
            if (vi * 16 < Cfg::A_BYTES) areg[q][r] = *reinterpret_cast<const v4i*>(wa + (size_t)vi * 16);
        }
    };
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
    auto store_lds = [&](int buf, int q) {
#pragma unroll
        for (int r = 0; r < Cfg::B_V; ++r) {
            const int j = j0 + r * J_STEP;
            v4i t;
            if constexpr (INF) t = v4i{quant4(bregf[q][r][0]), quant4(bregf[q][r][1]), quant4(bregf[q][r][2]), quant4(bregf[q][r][3])};
            else t = v4i{breg[q][r][0][0], breg[q][r][0][1], breg[q][r][1][0], breg[q][r][1][1]};
            *reinterpret_cast<v4i*>(&lds_b[buf][(j * TN + p_l) * 16]) = t;
        }
#pragma unroll
        for (int r = 0; r < Cfg::A_V; ++r) {
            const int vi = tid + r * 256;
            if (vi * 16 < Cfg::A_BYTES) *reinterpret_cast<v4i*>(&lds_a[buf][vi * 16]) = areg[q][r];
        }
    };

    v4i acc[FM][FN];

    // first: the accumulators start from the constant zero instead of being cleared beforehand
    auto multiply = [&](int buf, bool first) {
        v4i a[FM], b[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
            a[i] = *reinterpret_cast<const v4i*>(&lds_a[buf][((wm * FM + i) * 64 + lane) * 16]);
#pragma unroll
        for (int j = 0; j < FN; ++j)
            b[j] = *reinterpret_cast<const v4i*>(
                &lds_b[buf][((lane >> 4) * TN + wn * (TN / WN) + j * 16 + (lane & 15)) * 16]);
        if (first) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], v4i{0, 0, 0, 0}, 0, 0, 0);
        } else {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    };
    if constexpr (KC == 1) {
        load_global(0, 0);
        store_lds(0, 0);
        __syncthreads();
        for (int kc = 0; kc < n_chunks; ++kc) {
            const int buf = kc & 1;
            if (kc + 1 < n_chunks) load_global(kc + 1, 0);
            if (kc == 0) multiply(buf, true);
            else multiply(buf, false);
            if (kc + 1 < n_chunks) store_lds(buf ^ 1, 0);
            __syncthreads();
        }
    } else {
        // (the chunk tests are uniform over the workgroup)
#pragma unroll
        for (int q = 0; q < KC; ++q)
            if (q < n_chunks) load_global(q, q);
#pragma unroll
        for (int q = 0; q < KC; ++q)
            if (q < n_chunks) store_lds(q, q);
        __syncthreads();
        for (int k0 = 0; k0 < n_chunks; k0 += KC) {
            const int k1 = k0 + KC;  // first chunk of the next stage
#pragma unroll
            for (int q = 0; q < KC; ++q)
                if (k1 + q < n_chunks) load_global(k1 + q, q);
#pragma unroll
            for (int q = 0; q < KC; ++q)
                if (k0 + q < n_chunks) {
                    if (k0 + q == 0) multiply(q, true);
                    else multiply(q, false);
                }
            if (k1 < n_chunks) {
                __syncthreads();  // everyone has read this stage
#pragma unroll
                for (int q = 0; q < KC; ++q)
                    if (k1 + q < n_chunks) store_lds(q, q);
                __syncthreads();
            }
        }
    }
    // ---- epilogue -----------------------------------------------------------------------------------
    // (no `continue` / early exits inside the unrolled loops: the accumulator array must stay in registers)
    const int gq = lane >> 4;
    // image and pixel of this lane's first column; the other columns are 16, 32, ... pixels further: one division per
    // lane instead of one per column (a 32-bit division is ~20 vector instructions)
    const unsigned gp0 = tile_base + wn * (TN / WN) + (lane & 15);
    unsigned n0, pix0;
    locate((unsigned)(wn * (TN / WN) + (lane & 15)), n0, pix0);
    const bool wide = (unsigned)OHW >= 16u * FN;  // then a column is at most one image further than the first
    if constexpr (EPI == EPI_F32_P4 || EPI == EPI_F32_P4_FUSED || EPI == EPI_I8_P8 || EPI == EPI_I8_P8_NONNEG) {
        // Packed outputs. A lane's stores differ by a column offset (image, pixel) and a row
        // offset (channel group): each computed once, one 64-bit addition per store. LeakyReLU is decided once, in
        // front of the unrolled loops, not per value.
        constexpr bool FUSED = EPI == EPI_F32_P4_FUSED;  // plus the residual addend and / or the int8 twin
        constexpr bool F32 = EPI == EPI_F32_P4 || FUSED;
        constexpr int EB = F32 ? 16 : 8;       // bytes of one (pixel, channel group) element
        constexpr int CG = F32 ? 4 : 8;        // channels per group
        const size_t plane = (size_t)OHW * EB;  // one channel group of one image
        const size_t image = plane * (size_t)(Ks / CG);
        size_t col_ofs[FN];
        unsigned col_twin[FUSED ? FN : 1];  // the same for the Byte8 twin (below 2 GiB)
        bool col_ok[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const unsigned gpo = gp0 + j * 16;
            unsigned nn = n0, pp = pix0 + j * 16;
            if (wide) {
                if (pp >= (unsigned)OHW) pp -= (unsigned)OHW, ++nn;
            } else {
                nn = gpo / (unsigned)OHW;
                pp = gpo - nn * (unsigned)OHW;
            }
            col_ok[j] = gpo < total_pix;
            col_ofs[j] = (size_t)nn * image + (size_t)pp * EB;
            if constexpr (FUSED) col_twin[j] = (nn * (unsigned)(Ks / 8) * (unsigned)OHW + pp) * 8u;
        }
        auto rows = [&](auto lrelu_c) {
            constexpr bool LRELU = decltype(lrelu_c)::value;
#pragma unroll
            for (int ip = 0; ip < FM / 2; ++ip) {
                const int tpair = (mt0 + wm * FM) / 2 + ip;
                const int ch0 = 32 * tpair + 8 * gq;  // this lane's 8 consecutive output channels
                const bool ch_ok = ch0 < g.K;
                Epi8 prm;
                epi8_load<EPI>(prm, ep, ch0);  // arrays are padded to the padded rows
                const size_t row_ofs = (size_t)(ch0 / CG) * plane;
                char* row = (char*)out + row_ofs;
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    int a8[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        a8[e] = acc[2 * ip][j][e];
                        a8[4 + e] = acc[2 * ip + 1][j][e];
                    }
                    if (ch_ok && col_ok[j]) {
                        char* o = row + col_ofs[j];
                        if constexpr (FUSED) {
                            const size_t elem = (row_ofs + col_ofs[j]) >> 2;  // in floats, for the result and the addend
                            ohip_v2i tw = {0, 0};
                            tw[0] = (int)epi4_store_f32p4<true, LRELU ? 1 : 0>((float*)out, ep, prm.si, prm.bi, elem, a8[0], a8[1],
                                                                              a8[2], a8[3]);
                            if (ch0 + 4 < g.K)
                                tw[1] = (int)epi4_store_f32p4<true, LRELU ? 1 : 0>((float*)out, ep, prm.si + 4, prm.bi + 4,
                                                                                  elem + (plane >> 2), a8[4], a8[5], a8[6], a8[7]);
                            if (ep.twin != nullptr)  // K % 8 == 0 then: the lane's 8 channels are one Byte8 element
                                *reinterpret_cast<ohip_v2i*>(ep.twin + (size_t)(ch0 / 8) * OHW * 8 + col_twin[j]) = tw;
                        } else if constexpr (F32) {
                            *reinterpret_cast<ohip_v4i*>(o) =
                                epi4_dequant_f32p4<LRELU>(ep, prm.si, prm.bi, a8[0], a8[1], a8[2], a8[3]);
                            if (ch0 + 4 < g.K)
                                *reinterpret_cast<ohip_v4i*>(o + plane) =
                                    epi4_dequant_f32p4<LRELU>(ep, prm.si + 4, prm.bi + 4, a8[4], a8[5], a8[6], a8[7]);
                        } else {
                            *reinterpret_cast<ohip_v2i*>(o) =
                                epi8_quant_i8p8<EPI == EPI_I8_P8_NONNEG, LRELU ? 1 : 0>(ep, prm, a8);
                        }
                    }
                }
            }
        };
        if (EPI != EPI_I8_P8_NONNEG && ep.lrelu) rows(std::true_type{});
        else rows(std::false_type{});
    } else {
#pragma unroll
        for (int ip = 0; ip < FM / 2; ++ip) {
            const int tpair = (mt0 + wm * FM) / 2 + ip;
            const int ch0 = 32 * tpair + 8 * gq;  // this lane's 8 consecutive output channels
            const bool ch_ok = ch0 < g.K;
            Epi8 prm;
            if constexpr (EPI != EPI_GENERIC) epi8_load<EPI>(prm, ep, ch0);  // arrays are padded to the padded rows
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const unsigned gpo = gp0 + j * 16;
                int a8[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a8[e] = acc[2 * ip][j][e];
                    a8[4 + e] = acc[2 * ip + 1][j][e];
                }
                if (ch_ok && gpo < total_pix) {
                    unsigned nn = n0, pp = pix0 + j * 16;
                    if (wide) {
                        if (pp >= (unsigned)OHW) pp -= (unsigned)OHW, ++nn;
                    } else {
                        nn = gpo / (unsigned)OHW;
                        pp = gpo - nn * (unsigned)OHW;
                    }
                    const int n = (int)nn, pix = (int)pp;
                    {
                        epilogue_store8_generic(out, &ep, n, ch0, pix, g.K, OHW, a8[0], a8[1], a8[2], a8[3], a8[4], a8[5],
                                                a8[6], a8[7]);
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------

// weight rows are padded so that every kernel's row block is whole: 32, 64, or a multiple of 128
int igemm_padded_rows(int K) { return K <= 32 ? 32 : (K <= 64 ? 64 : (K + 127) / 128 * 128); }
int igemm_channel_groups(int C) { return (C + 63) / 64; }

// physical GEMM row -> logical output channel (rows of a pair of 16-row tiles are interleaved in fours, so
// that MFMA lane group q of the pair ends up with channels 32*pair + 8*q .. +7)
int igemm_row_channel(int row) {
    const int mt = row / 16, r = row % 16;
    return 32 * (mt / 2) + 8 * (r / 4) + 4 * (mt % 2) + (r % 4);
}

// how many kernel taps of a layer with C input channels fit one 64-deep reduction step (1: none are packed)
int igemm_tap_pack(int C, int kh, int kw) {
    if (kh * kw < 2) return 1;
    return C <= 16 ? 4 : (C <= 32 ? 2 : 1);
}

static int igemm_k_chunks(int C, int kh, int kw, int tap_pack) {
    return tap_pack > 1 ? (kh * kw + tap_pack - 1) / tap_pack : kh * kw * igemm_channel_groups(C);
}

size_t igemm_packed_weight_bytes(int K, int C, int kh, int kw, int tap_pack) {
    return (size_t)igemm_k_chunks(C, kh, kw, tap_pack) * (igemm_padded_rows(K) / 16) * 1024;
}

// weight [K, C, kh, kw] int8 -> [k-chunk = (tap, channel group)][16-row tile][lane][16 bytes]; with tap_pack > 1 a
// k-chunk is tap_pack taps: its 16-byte quarter j (= lane / 16) holds channels 16 (j % per) .. of tap tap_pack * kc + j / per
void igemm_pack_weights(const int8_t* w, int K, int C, int kh, int kw, int8_t* dst, int tap_pack) {
    const int mt16 = igemm_padded_rows(K) / 16, cgs = igemm_channel_groups(C);
    size_t o = 0;
    if (tap_pack > 1) {
        const int per = 4 / tap_pack;
        for (int kc = 0; kc < igemm_k_chunks(C, kh, kw, tap_pack); ++kc)
            for (int mt = 0; mt < mt16; ++mt)
                for (int lane = 0; lane < 64; ++lane) {
                    const int ch = igemm_row_channel(mt * 16 + (lane & 15));
                    const int j = lane >> 4, tap = kc * tap_pack + j / per;
                    for (int b = 0; b < 16; ++b, ++o) {
                        const int c = 16 * (j % per) + b;
                        dst[o] = (ch < K && c < C && tap < kh * kw) ? w[((size_t)ch * C + c) * kh * kw + tap] : 0;
                    }
                }
        return;
    }
    for (int tap = 0; tap < kh * kw; ++tap)
        for (int cg = 0; cg < cgs; ++cg)
            for (int mt = 0; mt < mt16; ++mt)
                for (int lane = 0; lane < 64; ++lane) {
                    const int ch = igemm_row_channel(mt * 16 + (lane & 15));
                    for (int b = 0; b < 16; ++b, ++o) {
                        const int c = cg * 64 + (lane >> 4) * 16 + b;
                        dst[o] = (ch < K && c < C) ? w[((size_t)ch * C + c) * kh * kw + tap] : 0;
                    }
                }
}

// k-chunks per stage of the staged variant: as many as keep a workgroup's LDS at 64 KB or less
template <int TM, int TN>
struct IgemmStage {
    static constexpr int KC = (TM + TN) * 64 * 4 <= 64 * 1024 ? 4 : 2;
};

template <int TM, int TN, int WM, int WN, int EPI, int KC>
static hipError_t launch_igemm_k(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                 hipStream_t stream) {
    const long total_pix = (long)g.N * g.OH * g.OW;
    const int n_pix_tiles = (int)((total_pix + TN - 1) / TN);
    const int mpad = igemm_padded_rows(g.K);
    const int m_tiles = (g.K + TM - 1) / TM;  // row blocks that hold at least one real channel (the rows are padded further)
    const int grid_z = g.Cs ? g.Cs / g.C : 1;  // groups of a grouped convolution
    hipLaunchKernelGGL((conv_igemm_kernel<TM, TN, WM, WN, EPI, KC>), dim3(n_pix_tiles, m_tiles, grid_z), dim3(256), 0,
                       stream, x, wpk, out, g, ep, mpad / 16, igemm_channel_groups(g.C), n_pix_tiles, (const float*)nullptr, 0.f);
    return hipGetLastError();
}

// the same launch on the fp32 Float8 blob of a pointwise layer (one k-chunk per stage)
template <int TM, int TN, int WM, int WN>
static hipError_t launch_igemm_f32in(const float* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                     const float* in_scale, float in_half, hipStream_t stream) {
    const long total_pix = (long)g.N * g.OH * g.OW;
    const int n_pix_tiles = (int)((total_pix + TN - 1) / TN);
    const int mpad = igemm_padded_rows(g.K);
    const dim3 grid(n_pix_tiles, (g.K + TM - 1) / TM, 1);
#define OHIP_IGF(E_)                                                                                                        \
    hipLaunchKernelGGL((conv_igemm_kernel<TM, TN, WM, WN, E_, 1, true>), grid, dim3(256), 0, stream, (const int8_t*)x, wpk, out, g, ep, \
                       mpad / 16, igemm_channel_groups(g.C), n_pix_tiles, in_scale, in_half)
    switch (pick_epilogue(ep, g.K)) {
    case EPI_I8_P8: OHIP_IGF(EPI_I8_P8); break;
    case EPI_I8_P8_NONNEG: OHIP_IGF(EPI_I8_P8_NONNEG); break;
    case EPI_F32_P4:
        if (ep.twin != nullptr || ep.residual != nullptr) OHIP_IGF(EPI_F32_P4_FUSED);
        else OHIP_IGF(EPI_F32_P4);
        break;
    default: return hipErrorInvalidValue;
    }
#undef OHIP_IGF
    return hipGetLastError();
}

template <int TM, int TN, int WM, int WN, int EPI>
static hipError_t launch_igemm_e(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                 int stage, hipStream_t stream) {
    // The staged variant shortens a workgroup's life (one global-memory latency per KC chunks) but needs KC times the
    // LDS. It pays when the whole grid is resident at once even so - the launch is then one workgroup life long -
    // and costs where the grid runs in rounds, which the smaller footprint packs tighter. (256 compute units.)
    const int n_chunks = igemm_k_chunks(g.C, g.kh, g.kw, g.tap_pack);
    bool staged = false;
    if (n_chunks >= 2) {
        constexpr int KCS = IgemmStage<TM, TN>::KC;
        const long per_cu = std::min<long>(4, (160 * 1024) / ((TM + TN) * 64 * KCS));
        const long wgs = ((long)g.N * g.OH * g.OW + TN - 1) / TN * ((g.K + TM - 1) / TM) * (g.Cs ? g.Cs / g.C : 1);
        staged = wgs <= per_cu * 256;
        if (stage) staged = stage == 2;  // forced by a test
    }
    if (staged) return launch_igemm_k<TM, TN, WM, WN, EPI, IgemmStage<TM, TN>::KC>(x, wpk, out, g, ep, stream);
    return launch_igemm_k<TM, TN, WM, WN, EPI, 1>(x, wpk, out, g, ep, stream);
}

template <int TM, int TN, int WM, int WN>
static hipError_t launch_igemm(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                               int stage, hipStream_t stream) {
    switch (pick_epilogue(ep, g.K)) {
    case EPI_I8_P8:
        return launch_igemm_e<TM, TN, WM, WN, EPI_I8_P8>(x, wpk, out, g, ep, stage, stream);
    case EPI_I8_P8_NONNEG:
        return launch_igemm_e<TM, TN, WM, WN, EPI_I8_P8_NONNEG>(x, wpk, out, g, ep, stage, stream);
    case EPI_F32_P4:
        if (ep.twin != nullptr || ep.residual != nullptr)
            return launch_igemm_e<TM, TN, WM, WN, EPI_F32_P4_FUSED>(x, wpk, out, g, ep, stage, stream);
        return launch_igemm_e<TM, TN, WM, WN, EPI_F32_P4>(x, wpk, out, g, ep, stage, stream);
    default:
        return launch_igemm_e<TM, TN, WM, WN, EPI_GENERIC>(x, wpk, out, g, ep, stage, stream);
    }
}

// tile choice. Long reductions (3x3 and larger over many channels): the widest row tile that does not pad M further,
// then a pixel tile of 128 where that still gives every compute unit work, else 64. Short reductions
// (pointwise layers, at most 16 k-chunks) are bound by latency and HBM: there the 128x256 tile's register count costs
// more occupancy than its reuse saves, and the tiles below were the fastest ones measured on MI355X over the pointwise
// shapes of a MobileNetV2 at batch 64 and 256->512 at 28x28.
void igemm_choose_tiles(const ConvGeom& g, int* tm, int* tn) {
    const int mpad = igemm_padded_rows(g.K);
    const long total_pix = (long)g.N * g.OH * g.OW;
    const int n_chunks = igemm_k_chunks(g.C, g.kh, g.kw, g.tap_pack);
    auto wgs = [&](int TM, int TN) { return ((total_pix + TN - 1) / TN) * ((g.K + TM - 1) / TM); };
    int TM = 32, TN = 64;
    if (n_chunks > 16) {
        if (mpad % 128 == 0) TM = 128;
        else if (mpad % 64 == 0) TM = 64;
        // measured over 3x3 / 5x5 layers of 64..512 channels at 14x14..112x112: 128 pixels beat 256 everywhere (the
        // wider tile halves the resident workgroups and its rounds quantise worse), 64 win below ~1.5 workgroups per CU
        if (wgs(TM, 128) >= 384) TN = 128;
    } else if (mpad >= 512 && mpad % 128 == 0) {
        TM = 128;
    } else if (mpad >= 64) {
        TM = 64;
        if (wgs(64, 256) >= 2048) TN = 256;
        else if (wgs(64, 128) >= 1024) TN = 128;
    } else {
        if (wgs(32, 256) >= 2048) TN = 256;
        else if (wgs(32, 128) >= 256) TN = 128;
    }
    *tm = TM;
    *tn = TN;
}

// A grouped (non-depthwise) convolution runs as one launch, a group per grid.z slice, when a group is whole octets of the
// input and whole elements of the output and the fast epilogues apply to a group's channel count.
bool igemm_grouped_applicable(const ConvGeom& g, const Epilogue& ep) {
    if (g.groups <= 1 || g.C % g.groups || g.K % g.groups || g.groups > 65535) return false;
    const int cg = g.C / g.groups, kg = g.K / g.groups;
    if (cg % 8) return false;
    const int epi = pick_epilogue(ep, kg);
    if (epi == EPI_GENERIC) return false;
    if (ep.twin != nullptr || ep.residual != nullptr) return false;
    return (epi == EPI_F32_P4) ? kg % 4 == 0 : kg % 8 == 0;
}

size_t igemm_grouped_weight_bytes(int K, int C, int groups, int kh, int kw) {
    return (size_t)groups * igemm_packed_weight_bytes(K / groups, C / groups, kh, kw, igemm_tap_pack(C / groups, kh, kw));
}

// weight [K, C/groups, kh, kw]: every group's [K/groups, C/groups, kh, kw] block packed by itself, one after the other
void igemm_pack_weights_grouped(const int8_t* w, int K, int C, int groups, int kh, int kw, int8_t* dst) {
    const int kg = K / groups, cg = C / groups;
    const int tp = igemm_tap_pack(cg, kh, kw);  // groups of at most 32 channels: two or four taps per reduction step
    const size_t per = igemm_packed_weight_bytes(kg, cg, kh, kw, tp);
    for (int grp = 0; grp < groups; ++grp)
        igemm_pack_weights(w + (size_t)grp * kg * cg * kh * kw, kg, cg, kh, kw, dst + grp * per, tp);
}

hipError_t run_conv_igemm(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g_in, const Epilogue& ep,
                          int tm, int tn, hipStream_t stream) {
    ConvGeom g = g_in;
    if (g.groups > 1) {  // one group's problem, the tensors' channel counts as strides
        if (!igemm_grouped_applicable(g_in, ep)) return hipErrorInvalidValue;
        g.Cs = g_in.C, g.Ks = g_in.K;
        g.C = g_in.C / g_in.groups, g.K = g_in.K / g_in.groups;
        g.groups = 1;
        g.tap_pack = igemm_tap_pack(g.C, g.kh, g.kw);  // (as igemm_pack_weights_grouped packed the weights)
    }
    // a forced pixel tile may carry the stage choice in its low bits (1: one chunk per stage, 2: the staged variant)
    const int stage = tn & 3;
    tn &= ~3;
    if (tm == 0 || tn == 0) igemm_choose_tiles(g, &tm, &tn);
    // a row tile must not reach past the padded weight rows
    if (igemm_padded_rows(g.K) % tm != 0) return hipErrorInvalidValue;
#define OHIP_IG(TM_, TN_, WM_, WN_) \
    if (tm == TM_ && tn == TN_) return launch_igemm<TM_, TN_, WM_, WN_>(x, wpk, out, g, ep, stage, stream);
    OHIP_IG(128, 256, 2, 2)
    OHIP_IG(128, 128, 2, 2)
    OHIP_IG(128, 64, 4, 1)
    OHIP_IG(64, 256, 2, 2)
    OHIP_IG(64, 128, 2, 2)
    OHIP_IG(64, 64, 2, 2)
    OHIP_IG(32, 256, 1, 4)
    OHIP_IG(32, 128, 1, 4)
    OHIP_IG(32, 64, 1, 4)
#undef OHIP_IG
    return hipErrorInvalidValue;
}

// true when run_conv_igemm_f32in takes this layer: a pointwise layer (1x1, stride 1, no padding, one group) on a Float8
// blob with one of the packed epilogues
bool igemm_f32in_applicable(const ConvGeom& g, const Epilogue& ep) {
    if (g.kh != 1 || g.kw != 1 || g.sh != 1 || g.sw != 1 || g.ph || g.pw || g.groups != 1 || g.C % 8) return false;
    const int epi = pick_epilogue(ep, g.K);
    if (epi != EPI_I8_P8 && epi != EPI_I8_P8_NONNEG && epi != EPI_F32_P4) return false;
    return (size_t)g.N * g.C * g.H * g.W * 4 < ((size_t)1 << 31);  // 32-bit byte offsets into the fp32 blob
}

hipError_t run_conv_igemm_f32in(const float* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                const float* in_scale, int in_round_mode, hipStream_t stream) {
    if (!igemm_f32in_applicable(g, ep)) return hipErrorInvalidValue;
    int tm, tn;
    igemm_choose_tiles(g, &tm, &tn);
    if (igemm_padded_rows(g.K) % tm != 0) return hipErrorInvalidValue;
    const float half = in_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
#define OHIP_IGF(TM_, TN_, WM_, WN_) \
    if (tm == TM_ && tn == TN_) return launch_igemm_f32in<TM_, TN_, WM_, WN_>(x, wpk, out, g, ep, in_scale, half, stream);
    OHIP_IGF(128, 64, 4, 1)
    OHIP_IGF(64, 256, 2, 2)
    OHIP_IGF(64, 128, 2, 2)
    OHIP_IGF(64, 64, 2, 2)
    OHIP_IGF(32, 256, 1, 4)
    OHIP_IGF(32, 128, 1, 4)
    OHIP_IGF(32, 64, 1, 4)
#undef OHIP_IGF
    return hipErrorInvalidValue;
}

}  // namespace ohip
