// A pointwise int8 -> int8 convolution and the depthwise 3x3 int8 -> int8 convolution that is its only reader, as one launch.
#include <algorithm>

#include "common.hpp"
#include "conv_dw_common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

// ---------------------------------------------------------------------------------------------------------------------
// A pointwise int8 -> int8 convolution followed by a depthwise 3x3 int8 -> int8 convolution that is its only reader (the
// first two layers of an inverted-residual block, Tensor/ConvolutionLayer.cpp:754-847 twice) in ONE launch: the expanded
// tensor -- six times the block's input in MobileNetV2 -- is never written to memory or read back; its rows exist only
// in LDS, as in conv_dw3x3_f32in_kernel above, whose walk this kernel shares.
//
// A wave owns 16 expanded channels (two octets) x the full image width x a strip of output rows. Per input row it
// computes the pointwise layer for its 16 channels on the matrix cores -- D[16 channels][16 pixels] per pixel group, the
// A operand (weights) in registers for the whole walk, the B operand (a pixel's input channels) straight from the Byte8
// blob, 8 bytes per lane (at most 32 input channels: v_mfma_i32_16x16x32_i8) or four 8-byte loads (at most 128: two
// reduction steps of v_mfma_i32_16x16x64_i8) -- requantizes the four channels a lane holds and writes them as one dword into the ring of
// LDS lines of their octet. Rows outside the image and pixels past the row's end are written as zeros: they are the
// depthwise layer's padding, not the pointwise layer's result on a zero input. The depthwise layer then reads its
// operands from those lines, octet by octet, exactly as conv_dw3x3_f32in_kernel does.
size_t xdw_weight_bytes(int Cin, int K) { return (size_t)(K / 16) * (Cin <= 32 ? 64 * 8 : 2 * 64 * 16); }

// weight [K][Cin] int8 -> A operands [K/16][reduction step][lane 64][16 bytes] (8 bytes for at most 32 input channels):
// lane (m = lane % 16, kq = lane / 16) holds row 16 pair + m, input channels 64 step + 16 kq .. + 15 (8 kq .. + 7)
void xdw_pack_weights(const int8_t* w, int Cin, int K, int8_t* dst) {
    std::fill(dst, dst + xdw_weight_bytes(Cin, K), (int8_t)0);
    const int steps = Cin <= 32 ? 1 : 2, per = Cin <= 32 ? 8 : 16;
    for (int pr = 0; pr < K / 16; ++pr)
        for (int ks = 0; ks < steps; ++ks)
            for (int lane = 0; lane < 64; ++lane)
                for (int b = 0; b < per; ++b) {
                    const int m = lane % 16, kq = lane / 16, c = 64 * ks + per * kq + b;
                    if (c < Cin) dst[(((size_t)pr * steps + ks) * 64 + lane) * per + b] = w[(size_t)(16 * pr + m) * Cin + c];
                }
}

template <int S, int EPI, bool XNN, int NG, int CK>
__global__ void __launch_bounds__(256, ((CK == 32 && (NG <= 4 || S == 2)) || (S == 2 && NG <= 4)) ? 3 : 2) conv_xdw_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wx,
                                                       const int8_t* __restrict__ wa, void* __restrict__ out, ConvGeom g, int cin,
                                                       Epilogue epx, Epilogue ep, int n_strips, int rps, unsigned in_bytes,
                                                       unsigned out_bytes) {
    constexpr int RL = 4, PF = 2;      // LDS lines per octet / rows of loads in flight
    constexpr int NCH = (NG + 3) / 4;  // column chunks of 64 pixels of the depthwise operand
    constexpr int T = S == 1 ? 2 : 1;  // A sets of the depthwise layer
    constexpr int PH = 4 / S;          // output pixels per lane column
    constexpr int KST = CK == 128 ? 2 : 1;
    constexpr int LINE = (64 * NCH + 8) * 8;
    constexpr int OCT = RL * LINE + 128;  // the second octet's lines, off the first one's banks
    extern __shared__ __attribute__((aligned(16))) int8_t lds_all[];  // [waves of the workgroup][2 octets][RL lines]
    const int C8 = g.C / 8, P = g.C / 16;
    unsigned bx = blockIdx.x, by = blockIdx.y;
    {  // consecutive strips of a plane and consecutive planes on one XCD (see conv_dw3x3_mfma_kernel)
        const unsigned id = by * gridDim.x + bx, total = gridDim.x * gridDim.y, per = total / 8;
        if (id < per * 8) {
            const unsigned w = (id % 8) * per + id / 8;
            bx = w % gridDim.x, by = w / gridDim.x;
        }
    }
    const int pr = by % P, img = by / P;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int strip = __builtin_amdgcn_readfirstlane(bx * (blockDim.x >> 6) + wave);
    if (strip >= n_strips) return;  // whole wave
    const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
    int8_t* const lds = lds_all + wave * (2 * OCT);

    // the padding slots of every line: pixels -2, -1 and 16 NG .. 64 NCH + 5 (the pixels from W to 16 NG - 1 are written
    // as zeros with every row)
    {
        constexpr int PADS = 64 * NCH + 8 - 16 * NG;
        for (int i = lane; i < PADS * RL * 2; i += 64) {
            const int line = i / PADS, k = i % PADS;
            const int slot = k < 2 ? k : 16 * NG + k;
            *reinterpret_cast<v2i*>(lds + (line / RL) * OCT + (line % RL) * LINE + slot * 8) = v2i{0, 0};
        }
    }

    // ---- pointwise layer: weights, this lane's input octet(s) of every pixel group, its four channels' constants -------
    const int Cin8 = cin / 8;
    const unsigned HW8 = (unsigned)(g.H * g.W) * 8u;
    const unsigned s_in = (unsigned)(img * Cin8) * HW8;
    const int oct0 = CK == 32 ? q : 2 * q;  // first input octet of this lane's reduction bytes
    unsigned v_in[NG];
#pragma unroll
    for (int p = 0; p < NG; ++p) v_in[p] = (16 * p + n < g.W && oct0 < Cin8) ? (unsigned)oct0 * HW8 + (unsigned)(16 * p + n) * 8u : DW_OOB;
    // (the other octets of this lane's reduction bytes: + 1, and + 8, + 9 in the second step; absent ones read zero)
    const bool ok1 = oct0 + 1 < Cin8, ok8 = oct0 + 8 < Cin8, ok9 = oct0 + 9 < Cin8;
    const __amdgpu_buffer_rsrc_t rin = dw_rsrc(x, in_bytes);
    const int oy0 = strip * rps;
    const int nrows = min(rps, g.OH - oy0);
    const int iy0 = oy0 * S - g.ph;
    const int nq = (nrows - 1) * S + 3;  // input rows this strip reads
    typedef v2i b_t[CK == 32 ? 1 : 2 * KST];
    auto issue = [&](int j, b_t (&dst)[NG]) {  // j: input row of the walk
        const int iy = iy0 + j;
        const bool ok = iy >= 0 && iy < g.H && j < nq;  // wave-uniform
        const unsigned s_row = (unsigned)__builtin_amdgcn_readfirstlane((int)(ok ? s_in + (unsigned)(iy * g.W) * 8u : 0u));
#pragma unroll
        for (int p = 0; p < NG; ++p) {
            const int vo = (int)(ok ? v_in[p] : DW_OOB);
            dst[p][0] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, vo, (int)s_row, 0));
            if constexpr (CK != 32) {
                dst[p][1] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, ok1 ? vo : (int)DW_OOB, (int)(s_row + HW8), 0));
                dst[p][2] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, ok8 ? vo : (int)DW_OOB, (int)(s_row + 8u * HW8), 0));
                dst[p][3] = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, ok9 ? vo : (int)DW_OOB, (int)(s_row + 9u * HW8), 0));
            }
        }
    };
    long ax32 = 0;
    v4i ax[KST];
    if constexpr (CK == 32) {
        ax32 = reinterpret_cast<const long*>(wx)[(size_t)pr * 64 + lane];
    } else {
#pragma unroll
        for (int ks = 0; ks < KST; ++ks) ax[ks] = reinterpret_cast<const v4i*>(wx)[((size_t)pr * KST + ks) * 64 + lane];
    }
    const int chx = 16 * pr + 4 * q;
    const v4i six = *reinterpret_cast<const v4i*>(epx.scale_in + chx);
    const v4i bix = *reinterpret_cast<const v4i*>(epx.bias + chx);
    const v4i sox = *reinterpret_cast<const v4i*>(epx.scale_out + chx);
    unsigned qx01 = 0, qx23 = 0;
    if constexpr (XNN) qx01 = dw_clamp_pair(epx, sox[0], sox[1]), qx23 = dw_clamp_pair(epx, sox[2], sox[3]);
    int8_t* const lds_w = lds + (q >> 1) * OCT + (n + 2) * 8 + 4 * (q & 1);  // this lane's dword of pixel group 0, line 0
    // the pointwise layer on input row j of the walk (in src) into LDS line `line` of both octets
    auto expand_write = [&](int j, int line, const b_t (&src)[NG]) {
        const int iy = iy0 + j;
        const unsigned rowm = (iy >= 0 && iy < g.H) ? 0xffffffffu : 0u;  // wave-uniform
        v4i d[NG];
#pragma unroll
        for (int p = 0; p < NG; ++p) {
            d[p] = v4i{0, 0, 0, 0};
            if constexpr (CK == 32) {
                d[p] = __builtin_amdgcn_mfma_i32_16x16x32_i8(ax32, __builtin_bit_cast(long, src[p][0]), d[p], 0, 0, 0);
            } else {
#pragma unroll
                for (int ks = 0; ks < KST; ++ks)
                    d[p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                        ax[ks], v4i{src[p][2 * ks][0], src[p][2 * ks][1], src[p][2 * ks + 1][0], src[p][2 * ks + 1][1]}, d[p], 0, 0, 0);
            }
        }
#pragma unroll
        for (int p = 0; p < NG; ++p) {
            unsigned w = dw_requant4<XNN>(epx, d[p], six, bix, sox, qx01, qx23) & rowm;
            if (16 * p + n >= g.W) w = 0;
            *reinterpret_cast<unsigned*>(lds_w + line * LINE + p * 128) = w;
        }
    };

    // ---- depthwise layer: weights and constants of both octets ---------------------------------------------------------
    v4i a[2][3][T];
#pragma unroll
    for (int oo = 0; oo < 2; ++oo) {
        const v4i* ap = reinterpret_cast<const v4i*>(wa) + (size_t)(2 * pr + oo) * 3 * T * 64 + lane;
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
            for (int t = 0; t < T; ++t) a[oo][k][t] = ap[(k * T + t) * 64];
    }
    __builtin_amdgcn_sched_barrier(0);

    b_t ld[PF][NG];
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(j, ld[j]);

    v4i si[2][T], bi[2][T], so[2][T];
    unsigned qh[2][T][2] = {};
#pragma unroll
    for (int oo = 0; oo < 2; ++oo) {
        const int ch = 8 * (2 * pr + oo) + (S == 1 ? 0 : 4 * (q & 1));
#pragma unroll
        for (int t = 0; t < T; ++t) {
            si[oo][t] = *reinterpret_cast<const v4i*>(ep.scale_in + ch + 4 * t);
            bi[oo][t] = *reinterpret_cast<const v4i*>(ep.bias + ch + 4 * t);
            so[oo][t] = *reinterpret_cast<const v4i*>(ep.scale_out + ch + 4 * t);
            // the bias is the fma's vector operand in every row: keep it resident (the compiler would otherwise re-copy
            // it from scalar registers value after value)
#pragma unroll
            for (int e = 0; e < 4; ++e) asm volatile("" : "+v"(bi[oo][t][e]));
            if constexpr (EPI == EPI_I8_P8_NONNEG) {
                qh[oo][t][0] = dw_clamp_pair(ep, so[oo][t][0], so[oo][t][1]);
                qh[oo][t][1] = dw_clamp_pair(ep, so[oo][t][2], so[oo][t][3]);
            }
        }
    }
    const unsigned OHW = (unsigned)(g.OH * g.OW);
    unsigned v_out[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int ox = PH * (16 * c + n) + (S == 1 ? q : (q >> 1));
        v_out[c] = ox < g.OW ? (unsigned)ox * 8u + (S == 1 ? 0u : (unsigned)(q & 1) * 4u) : DW_OOB;
    }
    const unsigned s_out = (unsigned)(img * C8 + 2 * pr) * OHW * 8u, row_bytes = (unsigned)g.OW * 8u;
    const __amdgpu_buffer_rsrc_t rout = dw_rsrc(out, out_bytes);

    v4i cur[2][NCH][T];
    auto epilogue_store = [&](int r) {  // output row r of the strip, from cur
        constexpr bool NONNEG = EPI == EPI_I8_P8_NONNEG;
#pragma unroll
        for (int oo = 0; oo < 2; ++oo) {
            const unsigned s_row =
                (unsigned)__builtin_amdgcn_readfirstlane((int)(s_out + (unsigned)oo * OHW * 8u + (unsigned)(oy0 + r) * row_bytes));
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                if constexpr (S == 1) {
                    v2i w2;
                    w2[0] = (int)dw_requant4<NONNEG>(ep, cur[oo][c][0], si[oo][0], bi[oo][0], so[oo][0], qh[oo][0][0], qh[oo][0][1]);
                    w2[1] = (int)dw_requant4<NONNEG>(ep, cur[oo][c][T - 1], si[oo][T - 1], bi[oo][T - 1], so[oo][T - 1], qh[oo][T - 1][0],
                                                     qh[oo][T - 1][1]);
                    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, w2), rout, (int)v_out[c], (int)s_row, 0);
                } else {
                    const unsigned w1 = dw_requant4<NONNEG>(ep, cur[oo][c][0], si[oo][0], bi[oo][0], so[oo][0], qh[oo][0][0], qh[oo][0][1]);
                    __builtin_amdgcn_raw_buffer_store_b32(w1, rout, (int)v_out[c], (int)s_row, 0);
                }
            }
        }
    };
    auto row_mfma = [&](int line0) {  // the three input rows of an output row sit in lines line0, +1, +2 (mod RL)
#pragma unroll
        for (int oo = 0; oo < 2; ++oo)
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                v4i b[3];
#pragma unroll
                for (int dy = 0; dy < 3; ++dy)
                    b[dy] = *reinterpret_cast<const v4i*>(lds + oo * OCT + ((line0 + dy) % RL) * LINE + (64 * c + 4 * n + 2 * q) * 8);
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    cur[oo][c][t] = v4i{0, 0, 0, 0};
#pragma unroll
                    for (int dy = 0; dy < 3; ++dy)
                        cur[oo][c][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[oo][dy][t], b[dy], cur[oo][c][t], 0, 0, 0);
                }
            }
    };
    // (the walk of conv_dw3x3_f32in_kernel: rows 0..2 in front of the loop, stores that go nowhere where there is no output
    // row to store yet, so that every path issues the same requests in the same order)
    auto no_store = [&](int i) {
#pragma unroll
        for (int oo = 0; oo < 2; ++oo)
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int nowhere = (int)(DW_OOB + 512u * (unsigned)i + 128u * (unsigned)oo + 64u * (unsigned)c);
                if constexpr (S == 1) __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, v2i{0, 0}), rout, nowhere, 0, 0);
                else __builtin_amdgcn_raw_buffer_store_b32(0u, rout, nowhere, 0, 0);
            }
    };
    auto input_row = [&](int j, int jj, bool store_prev) {  // jj = j modulo 4; a compile-time constant at every call
        expand_write(j, jj % RL, ld[jj % PF]);
        issue(j + PF, ld[jj % PF]);
        if ((jj - 2 + 4) % S == 0) {
            if (store_prev) epilogue_store((j - 2) / S - 1);
            else no_store(j);
            row_mfma((jj - 2 + 4) % RL);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    no_store(3);
    input_row(0, 0, false);
    input_row(1, 1, false);
    input_row(2, 2, false);
    constexpr int UNR = 8;
    const int steps = (nq - 3) / UNR;
    int jb = 3;
    for (int st = 0; st < steps; ++st, jb += UNR) {
#pragma unroll
        for (int i = 0; i < UNR; ++i) input_row(jb + i, 3 + i, true);
    }
#pragma unroll
    for (int i = 0; i < UNR - 1; ++i)
        if (jb + i < nq) input_row(jb + i, 3 + i, true);  // wave-uniform
    epilogue_store(nrows - 1);
}

// true when the two layers can run as conv_xdw_kernel (the caller has checked that both write int8 Byte8)
bool xdw_applicable(const ConvGeom& gx, const Epilogue& epx, int epi_x, bool sox_positive, const ConvGeom& gd, const Epilogue& ep,
                    int epi_d, bool so_positive) {
    if (gx.kh != 1 || gx.kw != 1 || gx.sh != 1 || gx.sw != 1 || gx.ph || gx.pw || gx.groups != 1) return false;
    if (gx.C % 8 || gx.C > 128 || gx.K % 16 || gx.K != gd.C) return false;
    if (gd.kh != 3 || gd.kw != 3 || gd.W > 128) return false;
    if (!dw_mfma_applicable(gd, ep, epi_d, so_positive)) return false;
    // both layers clamp at zero with positive output scales, or neither has a clamp beyond the int8 range
    const bool nn = epi_x == EPI_I8_P8_NONNEG && epi_d == EPI_I8_P8_NONNEG && sox_positive;
    const bool plain = epi_x == EPI_I8_P8 && epi_d == EPI_I8_P8;
    if (!nn && !plain) return false;
    (void)epx;
    if ((size_t)gx.N * gx.C * gx.H * gx.W >= ((size_t)1 << 31)) return false;  // 32-bit buffer offsets
    return (long)gd.N * (gd.C / 16) <= 65535;
}

hipError_t run_conv_xdw(const int8_t* x, const int8_t* wx, const int8_t* wa, void* out, const ConvGeom& gx, const Epilogue& epx,
                        const ConvGeom& g, const Epilogue& ep, int epi_d, int strip_rows, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const long planes = (long)g.N * (g.C / 16);
    if (planes > 65535) return hipErrorInvalidValue;
    // Strips of equal height. The kernel is bound by the vector instructions of its rows, so the launch lasts about as
    // long as the busiest of the chip's 1024 SIMDs: (waves per SIMD, rounded up) x (input rows a wave walks + about two
    // rows' worth of set-up). More strips balance the SIMDs better and recompute more halo rows; take the count that
    // minimises the product, the fewest strips among equals.
    int rps;
    if (strip_rows > 0) {
        rps = std::min(strip_rows, g.OH);
    } else {
        long best = -1;
        rps = g.OH;
        for (int r = g.OH; r >= 1; --r) {
            const int ns = (g.OH + r - 1) / r;
            const long per_simd = (planes * ns + 1023) / 1024;
            // (a lone wave issues a vector instruction every 6 cycles where two or more reach the pipe's 4)
            const long cost = per_simd * ((r - 1) * g.sh + 3 + 2) * (per_simd == 1 ? 15 : per_simd == 2 ? 11 : 10);
            if (best < 0 || cost < best) best = cost, rps = r;
        }
    }
    const int n_strips = (g.OH + rps - 1) / rps;
    const int wpb = n_strips % 4 == 0 ? 4 : (n_strips % 2 == 0 ? 2 : 1);
    const dim3 grid((unsigned)(n_strips / wpb), (unsigned)planes), block(64 * wpb);
    const int ng = (g.W + 15) / 16;
    const int NG = ng <= 1 ? 1 : (ng <= 2 ? 2 : (ng <= 4 ? 4 : (ng <= 7 ? 7 : 8)));
    const int nch = (NG + 3) / 4;
    const unsigned lds_bytes = (unsigned)wpb * 2u * (4u * (64u * nch + 8u) * 8u + 128u);
    const unsigned in_bytes = (unsigned)((size_t)gx.N * gx.C * gx.H * gx.W);
    const unsigned out_bytes = (unsigned)((size_t)g.N * g.K * g.OH * g.OW);
    const bool nn = epi_d == EPI_I8_P8_NONNEG;
#define OHIP_XDW_L(S_, NN_, G_, CK_)                                                                                              \
    hipLaunchKernelGGL((conv_xdw_kernel<S_, NN_ ? EPI_I8_P8_NONNEG : EPI_I8_P8, NN_, G_, CK_>), grid, block, lds_bytes, stream, x, wx, wa, \
                       out, g, gx.C, epx, ep, n_strips, rps, in_bytes, out_bytes)
#define OHIP_XDW_G(S_, NN_, CK_)                 \
    do {                                         \
        switch (NG) {                            \
        case 1: OHIP_XDW_L(S_, NN_, 1, CK_); break; \
        case 2: OHIP_XDW_L(S_, NN_, 2, CK_); break; \
        case 4: OHIP_XDW_L(S_, NN_, 4, CK_); break; \
        case 7: OHIP_XDW_L(S_, NN_, 7, CK_); break; \
        default: OHIP_XDW_L(S_, NN_, 8, CK_); break; \
        }                                        \
    } while (0)
#define OHIP_XDW_C(S_, NN_)                      \
    do {                                         \
        if (gx.C <= 32) OHIP_XDW_G(S_, NN_, 32); \
        else OHIP_XDW_G(S_, NN_, 128);           \
    } while (0)
    if (g.sh == 1) {
        if (nn) OHIP_XDW_C(1, true);
        else OHIP_XDW_C(1, false);
    } else {
        if (nn) OHIP_XDW_C(2, true);
        else OHIP_XDW_C(2, false);
    }
#undef OHIP_XDW_C
#undef OHIP_XDW_G
#undef OHIP_XDW_L
    return hipGetLastError();
}

}  // namespace ohip
