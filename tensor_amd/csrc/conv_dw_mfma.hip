// Depthwise 3x3 int8 convolution (stride 1 or 2, dilation 1, pad <= 1) on the reference's Byte8 layout, with the
// multiply-accumulate on the matrix cores.
//
// Why matrix cores for a layer with no channel reduction: with dot4 on the vector ALU the layer costs ~20 vector
// instructions per output value (9 dot4 + requantize) and is bound by the vector ALU at ~2x the time HBM needs.
// v_mfma_i32_16x16x64_i8 computes D[16 ch][16 px] += A[16 ch][64] * B[64][16 px]. Give the 64-deep reduction the
// meaning (column tap dx = 0..2 (+1 unused), channel j = 0..15) and let A be zero except A[i][(dx, i)] = w[i][dy][dx]:
// one instruction then does one kernel ROW of 16 channels x 16 pixels, three instructions do the 3x3 window, and the
// vector ALU is left with the requantize epilogue only. Three quarters of the multiplies are by zero; the matrix
// pipe has the room (it runs beside the vector ALU).
//
// The B operand needs no data movement beyond the load: lane (px = lane % 16, dx = lane / 16) supplies 16 reduction
// bytes = channels 0..15 of input pixel (row, px*S + dx - pad) = two 8-byte Byte8 elements from two adjacent channel
// octets. A lane's fragment of input row y serves kernel row 2 of output row y-2, row 1 of y-1 and row 0 of y (stride
// 1), so a wave walks down a strip of output rows, loading each input row once and keeping three in registers.
// Image borders cost no instructions: loads and stores go through buffer descriptors, a lane that falls outside
// the image (or outside the channel count) carries an out-of-range offset, reads zero and writes nothing.
#include <algorithm>

#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

// weight [C, 1, 3, 3] int8 -> A operands [C/16 groups][kernel row 3][lane 64][16 bytes]:
// lane (i = lane % 16, dx = lane / 16) holds w[16*group + i][row][dx] in byte i, zero elsewhere
size_t dw_mfma_weight_bytes(int C) { return (size_t)((C + 15) / 16) * 3 * 64 * 16; }

void dw_mfma_pack_weights(const int8_t* w, int C, int8_t* dst) {
    std::fill(dst, dst + dw_mfma_weight_bytes(C), (int8_t)0);
    for (int c = 0; c < C; ++c)
        for (int dy = 0; dy < 3; ++dy)
            for (int dx = 0; dx < 3; ++dx) {
                const int grp = c / 16, i = c % 16, lane = dx * 16 + i;
                dst[(((size_t)grp * 3 + dy) * 64 + lane) * 16 + i] = w[(size_t)c * 9 + dy * 3 + dx];
            }
}

constexpr unsigned DW_OOB = 0x80000000u;  // beyond any descriptor this file builds (tensors are kept below 2 GiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dw_rsrc(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// A wave owns 16 output columns x 16 channels and walks down `rps` output rows. The input rows live in a ring of 8
// register fragments: a step computes 8/S output rows from the ring and refills every slot as soon as its last reader
// has issued, so the loads run 5 input rows ahead of the matrix instructions for the whole walk.
template <int S, int EPI>
__global__ void __launch_bounds__(256) conv_dw3x3_mfma_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wa,
                                                              void* __restrict__ out, ConvGeom g, Epilogue ep,
                                                              int n_strips, int rps, int col_chunks, int ipw,
                                                              unsigned in_bytes, unsigned out_bytes) {
    constexpr int RING = 8, U = RING / S;  // output rows per step
    const int C8 = g.C / 8, G16 = (C8 + 1) / 2;
    const int grp = blockIdx.y % G16;
    const int n0 = (blockIdx.y / G16) * ipw;
    const int chunk = blockIdx.x % col_chunks;
    const int strip = __builtin_amdgcn_readfirstlane((blockIdx.x / col_chunks) * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (strip >= n_strips) return;  // whole wave
    const int lane = threadIdx.x & 63, px = lane & 15, q = lane >> 4;
    // 16 output columns per wave; images of at most 8 columns sit side by side (same channels, consecutive images)
    int di = 0, ox = chunk * 16 + px;
    if (ipw > 1) {
        di = px / g.OW;
        ox = px - di * g.OW;
    }
    const bool lane_ok = ox < g.OW && di < ipw && n0 + di < g.N;
    const bool has_hi = 2 * grp + 1 < C8;  // the group's second octet exists (C % 16 == 8 ends on a single octet)

    // ---- input: per-lane byte offset (fixed for the whole walk) + per-row scalar offset -------------------------
    const unsigned HW8 = (unsigned)(g.H * g.W * 8);
    const int ix = ox * S - g.pw + q;
    const bool col_ok = lane_ok && q < 3 && ix >= 0 && ix < g.W;
    const unsigned v_lo = col_ok ? (unsigned)di * (unsigned)C8 * HW8 + (unsigned)ix * 8u : DW_OOB;
    const unsigned v_hi = (col_ok && has_hi) ? v_lo + HW8 : DW_OOB;
    const unsigned s_in = (unsigned)(n0 * C8 + 2 * grp) * HW8;
    const __amdgpu_buffer_rsrc_t rin = dw_rsrc(x, in_bytes);

    const int oy0 = strip * rps;
    const int iy0 = oy0 * S - g.ph;
    const int rows_needed = (min(rps, g.OH - oy0) - 1) * S + 3;  // input rows this strip really reads
    auto load_row = [&](int j) -> v4i {  // j: input row relative to iy0; rows outside the image or the strip read zero
        const int iy = iy0 + j;
        const bool ok = iy >= 0 && iy < g.H && j < rows_needed;  // wave-uniform
        const unsigned s_row = ok ? s_in + (unsigned)(iy * g.W * 8) : 0u;
        const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(ok ? v_lo : DW_OOB), (int)s_row, 0));
        const v2i hi = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(ok ? v_hi : DW_OOB), (int)s_row, 0));
        return v4i{lo[0], lo[1], hi[0], hi[1]};
    };

    v4i frag[RING];
#pragma unroll
    for (int j = 0; j < RING; ++j) frag[j] = load_row(j);

    const v4i* ap = reinterpret_cast<const v4i*>(wa) + (size_t)grp * 3 * 64 + lane;
    const v4i a0 = ap[0], a1 = ap[64], a2 = ap[128];

    // ---- epilogue constants of this lane's four channels 16*grp + 4*q .. +3 (arrays are padded past K) ---------
    const int ch = 16 * grp + 4 * q;
    const v4i si4 = *reinterpret_cast<const v4i*>(ep.scale_in + ch);
    const v4i bi4 = *reinterpret_cast<const v4i*>(ep.bias + ch);
    v4i so4 = {0, 0, 0, 0};
    if constexpr (EPI != EPI_F32_P4) so4 = *reinterpret_cast<const v4i*>(ep.scale_out + ch);

    // ---- output: same scheme --------------------------------------------------------------------------------
    const unsigned OHW = (unsigned)(g.OH * g.OW);
    const bool st_ok = lane_ok && (q < 2 || has_hi);
    unsigned v_out, s_out, row_bytes;
    if constexpr (EPI == EPI_F32_P4) {  // Float4: [N][C/4][OH*OW][4 floats]; this lane's channels are pack 4*grp + q
        v_out = st_ok ? ((unsigned)di * (unsigned)(g.C / 4) + (unsigned)q) * OHW * 16u + (unsigned)ox * 16u : DW_OOB;
        s_out = (unsigned)(n0 * (g.C / 4) + 4 * grp) * OHW * 16u;
        row_bytes = (unsigned)g.OW * 16u;
    } else {  // Byte8: [N][C/8][OH*OW][8 bytes]; octet 2*grp + q/2, bytes 4*(q%2)..+3
        v_out = st_ok ? ((unsigned)di * (unsigned)C8 + (unsigned)(q >> 1)) * OHW * 8u + (unsigned)ox * 8u + (unsigned)(q & 1) * 4u
                      : DW_OOB;
        s_out = (unsigned)(n0 * C8 + 2 * grp) * OHW * 8u;
        row_bytes = (unsigned)g.OW * 8u;
    }
    const __amdgpu_buffer_rsrc_t rout = dw_rsrc(out, out_bytes);

    for (int rb = 0; rb < rps; rb += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int oy = oy0 + rb + u;
            v4i acc = {0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, frag[(u * S + 0) % RING], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, frag[(u * S + 1) % RING], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, frag[(u * S + 2) % RING], acc, 0, 0, 0);
            // the S oldest rows are dead now: refill their slots with the rows one ring ahead
#pragma unroll
            for (int k = 0; k < S; ++k) frag[(u * S + k) % RING] = load_row((rb + u) * S + k + RING);
            const bool row_ok = oy < g.OH && rb + u < rps;  // rows past the strip / image are dropped
            const unsigned s_row = row_ok ? s_out + (unsigned)oy * row_bytes : 0u;
            const unsigned v_o = row_ok ? v_out : DW_OOB;
            if constexpr (EPI == EPI_F32_P4) {
                v4i res;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = __fmaf_rn((float)acc[e], __int_as_float(si4[e]), __int_as_float(bi4[e]));
                    v = fminf(fmaxf(v, ep.act_lo), ep.act_hi);
                    res[e] = __float_as_int(v);
                }
                __builtin_amdgcn_raw_buffer_store_b128(
                    __builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, res), rout, (int)v_o,
                    (int)s_row, 0);
            } else {
                constexpr bool NONNEG = EPI == EPI_I8_P8_NONNEG;
                int qv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = __fmaf_rn((float)acc[e], __int_as_float(si4[e]), __int_as_float(bi4[e]));
                    v = __builtin_amdgcn_fmed3f(v, ep.act_lo, ep.act_hi);
                    v = __fmul_rn(v, __int_as_float(so4[e]));
                    const float adj =
                        NONNEG ? __fadd_rn(v, ep.round_half) : __fadd_rn(v, __builtin_copysignf(ep.round_half, v));
                    qv[e] = (int)adj;  // toward zero, saturating
                }
                ohip_v2s lo = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(qv[0], qv[1]));
                ohip_v2s hi = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(qv[2], qv[3]));
                const ohip_v2s top = {127, 127}, bot = {-127, -127};
                lo = __builtin_elementwise_min(lo, top);
                hi = __builtin_elementwise_min(hi, top);
                if (!NONNEG) {
                    lo = __builtin_elementwise_max(lo, bot);
                    hi = __builtin_elementwise_max(hi, bot);
                }
                const unsigned word =
                    __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
                __builtin_amdgcn_raw_buffer_store_b32(word, rout, (int)v_o, (int)s_row, 0);
            }
        }
    }
}

// true when this layer / batch can take the matrix-core kernel (the caller falls back to the vector kernels otherwise)
bool dw_mfma_applicable(const ConvGeom& g, const Epilogue& ep, int epi) {
    if (!(g.kh == 3 && g.kw == 3 && g.dh == 1 && g.dw == 1 && g.sh == g.sw && (g.sh == 1 || g.sh == 2))) return false;
    if (g.ph > 1 || g.pw > 1 || g.C % 8 != 0 || g.C != g.K) return false;
    if (epi != EPI_I8_P8 && epi != EPI_I8_P8_NONNEG && epi != EPI_F32_P4) return false;
    const size_t in_bytes = (size_t)g.N * g.C * g.H * g.W;
    const size_t out_bytes = (size_t)g.N * g.K * g.OH * g.OW * (epi == EPI_F32_P4 ? 4 : 1);
    return in_bytes < ((size_t)1 << 31) && out_bytes < ((size_t)1 << 31);  // 32-bit buffer offsets
}

hipError_t run_conv_dw_mfma(const int8_t* x, const int8_t* wa, void* out, const ConvGeom& g, const Epilogue& ep, int epi,
                            int strip_blocks, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const int G16 = (g.C / 8 + 1) / 2;
    const int col_chunks = (g.OW + 15) / 16;
    const int ipw = g.OW <= 8 ? std::min(16 / g.OW, g.N) : 1;
    const long groups = (long)((g.N + ipw - 1) / ipw) * G16;
    if (groups > 65535) return hipErrorInvalidValue;  // grid.y limit; the caller splits the batch
    // strip height in steps of U = 8/stride output rows: the tallest strip (setup and halo rows amortised over the
    // longest walk) that still leaves about four waves per SIMD
    const int U = 8 / g.sh;
    const int blocks_total = (g.OH + U - 1) / U;
    int k = blocks_total;
    if (strip_blocks > 0) k = std::min(strip_blocks, blocks_total);
    else
        while (k > 1 && (long)col_chunks * ((blocks_total + k - 1) / k) * groups < 4096) --k;
    const int rps = k * U;
    const int n_strips = (g.OH + rps - 1) / rps;
    const int wpb = n_strips % 4 == 0 ? 4 : (n_strips % 2 == 0 ? 2 : 1);
    const dim3 grid((unsigned)(col_chunks * (n_strips / wpb)), (unsigned)groups), block(64 * wpb);
    const unsigned in_bytes = (unsigned)((size_t)g.N * g.C * g.H * g.W);
    const unsigned out_bytes = (unsigned)((size_t)g.N * g.K * g.OH * g.OW * (epi == EPI_F32_P4 ? 4 : 1));
#define OHIP_DWM(S_, E_)                                                                                               \
    hipLaunchKernelGGL((conv_dw3x3_mfma_kernel<S_, E_>), grid, block, 0, stream, x, wa, out, g, ep, n_strips, rps, col_chunks, \
                       ipw, in_bytes, out_bytes)
#define OHIP_DWM_E(S_)                                                \
    do {                                                              \
        if (epi == EPI_I8_P8_NONNEG) OHIP_DWM(S_, EPI_I8_P8_NONNEG);  \
        else if (epi == EPI_I8_P8) OHIP_DWM(S_, EPI_I8_P8);           \
        else OHIP_DWM(S_, EPI_F32_P4);                                \
    } while (0)
    if (g.sh == 1) OHIP_DWM_E(1);
    else OHIP_DWM_E(2);
#undef OHIP_DWM_E
#undef OHIP_DWM
    return hipGetLastError();
}

}  // namespace ohip
