// Depthwise 3x3 int8 convolution (stride 1 or 2, dilation 1, pad <= 1) on the reference's Byte8 layout, with the
// multiply-accumulate on the matrix cores.
//
// Why matrix cores for a layer with no channel reduction: with dot4 on the vector ALU the layer costs ~20 vector
// instructions per output value (9 dot4 + requantize) and is bound by the vector ALU at ~2x the time HBM needs.
// v_mfma_i32_16x16x64_i8 computes D[16][16] += A[16][64] * B[64][16]. Here a B column n is a run of 4 output pixels
// (stride 1; 2 for stride 2) of one channel octet, and its 64 reduction bytes are the 8 input pixels 4n-2 .. 4n+5 of
// one input row x 8 channels: lane (n, g = lane / 16) supplies pixels 4n-2+2g and +1, i.e. ONE aligned 16-byte load.
// A D row m is (output pixel phase p, channel c) and A is zero except A[(p, c)][(pixel e, channel c)] = w[c][dy][dx]
// for the dx that connects input pixel e to output phase p. One instruction does one kernel ROW for 16 x 16 (phase,
// channel, column) outputs, three do the 3x3 window, and the vector ALU is left with the requantize epilogue only.
// Most multiplies are by zero; the matrix pipe has the room (it runs beside the vector ALU).
//
// Stride 1: two A sets (channels 0-3 and 4-7 of the octet) share the B fragment; a lane ends up with all 8 channels
// of output pixel 4n + lane/16 and stores one Byte8 element. Stride 2: one A set, rows = 2 phases x 8 channels; a
// lane ends up with 4 channels of output pixel 2n + lane/32.
// A lane's fragment of input row y serves kernel row 2 of output row y-2, row 1 of y-1 and row 0 of y (stride 1),
// so a wave walks down a strip of output rows with the input rows in a ring of registers, each loaded once.
// Image borders cost no instructions: loads and stores go through buffer descriptors, a lane that falls outside
// the image carries an out-of-range offset, reads zero and writes nothing.
#include <algorithm>

#include "common.hpp"
#include "conv_dw_common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

// weight [C, 1, ks, ks] int8 (ks = 3 or 5) -> A operands [C/8 octets][kernel row ks][set T][lane 64][16 bytes], T = 2 for stride 1
// (set t = channels 4t..4t+3) and 1 for stride 2. Lane (r = lane % 16, g = lane / 16) holds A[row r][16g .. 16g+15];
// reduction byte 16g + 8e + j is (input pixel 4n-2+2g+e, channel j).
static int dw_mfma_sets(int stride) { return stride == 1 ? 2 : 1; }
size_t dw_mfma_weight_bytes(int C, int stride, int ks) { return (size_t)(C / 8) * ks * dw_mfma_sets(stride) * 64 * 16; }

// The 8 input pixels 4n-2 .. 4n+5 of a column must cover the windows of its 4 (stride 1) or 2 (stride 2) outputs:
// with pad_w columns of padding the window of output phase p starts at pixel slot 2 + stride*p - pad_w.
bool dw_mfma_window_fits(int ks, int stride, int pad_w) {
    const int phases = 4 / stride;
    return 2 - pad_w >= 0 && (ks - 1) + 2 + stride * (phases - 1) - pad_w <= 7;
}

void dw_mfma_pack_weights(const int8_t* w, int C, int stride, int pad_w, int ks, int8_t* dst) {
    const int T = dw_mfma_sets(stride);
    std::fill(dst, dst + dw_mfma_weight_bytes(C, stride, ks), (int8_t)0);
    for (int o = 0; o < C / 8; ++o)
        for (int dy = 0; dy < ks; ++dy)
            for (int t = 0; t < T; ++t)
                for (int lane = 0; lane < 64; ++lane) {
                    const int r = lane % 16, g = lane / 16;
                    // D row r -> (output pixel phase p, channel c of the octet)
                    const int p = stride == 1 ? r / 4 : r / 8;
                    const int c = stride == 1 ? 4 * t + r % 4 : r % 8;
                    for (int e = 0; e < 2; ++e) {
                        // input pixel 4n - 2 + 2g + e feeds output pixel (4/stride) n + p through tap dx
                        const int dx = 2 * g + e - 2 - stride * p + pad_w;
                        if (dx < 0 || dx >= ks) continue;
                        dst[((((size_t)o * ks + dy) * T + t) * 64 + lane) * 16 + 8 * e + c] =
                            w[(size_t)(8 * o + c) * ks * ks + dy * ks + dx];
                    }
                }
}

__device__ __forceinline__ v4i dw_dequant4(const Epilogue& ep, const v4i& acc, const v4i& si, const v4i& bi) {
    v4i res;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = __fmaf_rn((float)acc[e], __int_as_float(si[e]), __int_as_float(bi[e]));
        v = fminf(fmaxf(v, ep.act_lo), ep.act_hi);
        if (ep.lrelu) v = fmaxf(v, __fmul_rn(v, ep.act_p0));  // wave-uniform branch; the clamp above is open then
        res[e] = __float_as_int(v);
    }
    return res;
}

// A wave owns one channel octet x 16 lane columns (64 output pixels of a row at stride 1, 32 at stride 2) and walks
// down `rps` output rows. The input rows live in a ring of 8 register fragments: a step computes 8/S output rows
// from the ring and refills every slot as soon as its last reader has issued, so the loads run 5 input rows ahead of
// the matrix instructions for the whole walk. Narrow images sit side by side in the wave (`lpi` lane columns each).
template <int S, int EPI, bool ODDW, int KS>
__global__ void __launch_bounds__(256) conv_dw3x3_mfma_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wa,
                                                              void* __restrict__ out, ConvGeom g, Epilogue ep,
                                                              int n_strips, int rps, int col_chunks, int lpi, int ipw,
                                                              unsigned in_bytes, unsigned out_bytes) {
    constexpr int RING = 8, U = RING / S;  // U output rows per step
    constexpr int PH = 4 / S;              // output pixels per lane column
    constexpr int T = S == 1 ? 2 : 1;      // A sets
    const int C8 = g.C / 8;
    // Workgroups go to the 8 XCDs round-robin in launch order. Work items that share input cache lines - the column
    // chunks of a row (a 128-byte line straddles the chunk border), the strip groups of a plane (halo rows), the
    // octets of an image - get consecutive indices on ONE XCD, so that a shared line comes from memory once.
    unsigned bx = blockIdx.x, by = blockIdx.y;
    {
        const unsigned id = by * gridDim.x + bx, total = gridDim.x * gridDim.y, per = total / 8;
        if (id < per * 8) {
            const unsigned w = (id % 8) * per + id / 8;
            bx = w % gridDim.x, by = w / gridDim.x;
        }
    }
    const int o = by % C8;
    const int n0 = (by / C8) * ipw;
    const int chunk = bx % col_chunks;
    const int strip = __builtin_amdgcn_readfirstlane((bx / col_chunks) * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (strip >= n_strips) return;  // whole wave
    const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
    int di = 0, nl = chunk * 16 + n;  // image within the wave, lane column within the image
    if (ipw > 1) {
        di = n / lpi;
        nl = n - di * lpi;
    }
    const bool lane_ok = di < ipw && n0 + di < g.N;

    // ---- input: one 16-byte load per lane and row; per-lane byte offset fixed for the walk + per-row scalar offset --
    const unsigned HW8 = (unsigned)(g.H * g.W * 8);
    const int ic = 4 * nl - 2 + 2 * q;  // first input pixel of this lane's pair
    const bool in_ok = lane_ok && ic >= 0 && ic < g.W;
    const unsigned v_in = in_ok ? (unsigned)di * (unsigned)C8 * HW8 + (unsigned)ic * 8u : DW_OOB;
    const unsigned v_in2 = (in_ok && ic + 1 < g.W) ? v_in + 8u : DW_OOB;  // second pixel of the pair (odd widths only)
    const unsigned s_in = (unsigned)(n0 * C8 + o) * HW8;
    const __amdgpu_buffer_rsrc_t rin = dw_rsrc(x, in_bytes);

    const int oy0 = strip * rps;
    const int iy0 = oy0 * S - g.ph;
    const int rows_needed = (min(rps, g.OH - oy0) - 1) * S + KS;  // input rows this strip really reads
    auto load_row = [&](int j) -> v4i {  // j: input row relative to iy0; rows outside the image or the strip read zero
        const int iy = iy0 + j;
        const bool ok = iy >= 0 && iy < g.H && j < rows_needed;  // wave-uniform
        const unsigned s_row = ok ? s_in + (unsigned)(iy * g.W * 8) : 0u;
        if constexpr (ODDW) {  // odd width: a row ends on half a pair, which is loaded as 8 bytes + zero
            const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(ok ? v_in : DW_OOB), (int)s_row, 0));
            const v2i hi = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)(ok ? v_in2 : DW_OOB), (int)s_row, 0));
            return v4i{lo[0], lo[1], hi[0], hi[1]};
        }
        const v4i f = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(ok ? v_in : DW_OOB), (int)s_row, 0));
        return f;
    };

    v4i frag[RING];
#pragma unroll
    for (int j = 0; j < RING; ++j) frag[j] = load_row(j);

    v4i a[KS][T];
    {
        const v4i* ap = reinterpret_cast<const v4i*>(wa) + (size_t)o * KS * T * 64 + lane;
#pragma unroll
        for (int dy = 0; dy < KS; ++dy)
#pragma unroll
            for (int t = 0; t < T; ++t) a[dy][t] = ap[(dy * T + t) * 64];
    }

    // ---- epilogue constants: stride 1 -> the octet's 8 channels (same for every lane); stride 2 -> this lane's 4 ----
    const int ch = 8 * o + (S == 1 ? 0 : 4 * (q & 1));
    v4i si[T], bi[T], so[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        si[t] = *reinterpret_cast<const v4i*>(ep.scale_in + ch + 4 * t);
        bi[t] = *reinterpret_cast<const v4i*>(ep.bias + ch + 4 * t);
        so[t] = v4i{0, 0, 0, 0};
        if constexpr (EPI != EPI_F32_P4 && EPI != EPI_F32_P8) so[t] = *reinterpret_cast<const v4i*>(ep.scale_out + ch + 4 * t);
        // the bias is the fma's vector operand in every row: keep it resident (the compiler would otherwise re-copy
        // it from scalar registers row after row)
#pragma unroll
        for (int e = 0; e < 4; ++e) asm volatile("" : "+v"(bi[t][e]));
    }
    unsigned qh[T][2] = {};
    if constexpr (EPI == EPI_I8_P8_NONNEG) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
            qh[t][0] = dw_clamp_pair(ep, so[t][0], so[t][1]);
            qh[t][1] = dw_clamp_pair(ep, so[t][2], so[t][3]);
        }
    }

    // ---- output: this lane's pixel of the row, same addressing scheme ----------------------------------------------
    const unsigned OHW = (unsigned)(g.OH * g.OW);
    const int ox = PH * nl + (S == 1 ? q : (q >> 1));
    const bool st_ok = lane_ok && ox < g.OW;
    unsigned v_out, s_out, row_bytes;
    if constexpr (EPI == EPI_F32_P4) {  // Float4: [N][C/4][OH*OW][4 floats]; packs 2o and 2o+1
        v_out = st_ok ? ((unsigned)di * (unsigned)(g.C / 4) + (S == 1 ? 0u : (unsigned)(q & 1))) * OHW * 16u + (unsigned)ox * 16u
                      : DW_OOB;
        s_out = (unsigned)(n0 * (g.C / 4) + 2 * o) * OHW * 16u;
        row_bytes = (unsigned)g.OW * 16u;
    } else if constexpr (EPI == EPI_F32_P8) {  // Float8: [N][C/8][OH*OW][8 floats]; a lane's sets are the pixel's halves
        v_out = st_ok ? (unsigned)di * (unsigned)C8 * OHW * 32u + (unsigned)ox * 32u + (S == 1 ? 0u : (unsigned)(q & 1) * 16u)
                      : DW_OOB;
        s_out = (unsigned)(n0 * C8 + o) * OHW * 32u;
        row_bytes = (unsigned)g.OW * 32u;
    } else {  // Byte8: [N][C/8][OH*OW][8 bytes]
        v_out = st_ok ? (unsigned)di * (unsigned)C8 * OHW * 8u + (unsigned)ox * 8u + (S == 1 ? 0u : (unsigned)(q & 1) * 4u)
                      : DW_OOB;
        s_out = (unsigned)(n0 * C8 + o) * OHW * 8u;
        row_bytes = (unsigned)g.OW * 8u;
    }
    const __amdgpu_buffer_rsrc_t rout = dw_rsrc(out, out_bytes);

    // Software pipeline, one output row deep: a step issues the matrix instructions of row r+1, refills the ring slots
    // they free, and then runs the epilogue of row r while those instructions execute. The scheduling barriers keep
    // the compiler from batching all matrix instructions at the top of the loop (which exposes the load latency).
    auto row_mfma = [&](int u, v4i (&acc)[T]) {  // u: output row within the step (ring phase)
#pragma unroll
        for (int t = 0; t < T; ++t) {
            acc[t] = v4i{0, 0, 0, 0};
#pragma unroll
            for (int dy = 0; dy < KS; ++dy)
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[dy][t], frag[(u * S + dy) % RING], acc[t], 0, 0, 0);
        }
    };
    v4i cur[T], nxt[T];
    row_mfma(0, cur);
#pragma unroll
    for (int k = 0; k < S; ++k) frag[k % RING] = load_row(k + RING);
    __builtin_amdgcn_sched_barrier(0);

    auto epilogue_store = [&](unsigned v_o, unsigned s_row, bool row_ok) {
        if constexpr (EPI == EPI_F32_P4 || EPI == EPI_F32_P8) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const v4i res = dw_dequant4(ep, cur[t], si[t], bi[t]);
                // the second set's channels 4..7: the next Float4 pack is one plane further, in Float8 they follow
                const unsigned vo_t = (t == 0 || !row_ok) ? v_o : v_o + (EPI == EPI_F32_P4 ? OHW * 16u : 16u);
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_store, res), rout, (int)vo_t, (int)s_row, 0);
            }
        } else {
            constexpr bool NONNEG = EPI == EPI_I8_P8_NONNEG;
            if constexpr (S == 1) {
                v2i w2;
                w2[0] = (int)dw_requant4<NONNEG>(ep, cur[0], si[0], bi[0], so[0], qh[0][0], qh[0][1]);
                w2[1] = (int)dw_requant4<NONNEG>(ep, cur[T - 1], si[T - 1], bi[T - 1], so[T - 1], qh[T - 1][0], qh[T - 1][1]);
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, w2), rout, (int)v_o, (int)s_row, 0);
            } else {
                const unsigned w1 = dw_requant4<NONNEG>(ep, cur[0], si[0], bi[0], so[0], qh[0][0], qh[0][1]);
                __builtin_amdgcn_raw_buffer_store_b32(w1, rout, (int)v_o, (int)s_row, 0);
            }
        }
    };

    // A step of U rows is "interior" when every row it stores lies inside the strip and every row it loads inside
    // the image: then the per-row scalar offsets just advance and nothing is predicated. The steps at the
    // end of a strip take the checked path, which also leaves as soon as the strip's last row is stored (a strip need
    // not be a whole number of steps).
    const int nrows = min(rps, g.OH - oy0);
    // loads of rows [RING, in_rows_ok) stay inside the image (iy0 + RING > 0); the few an interior step fetches past
    // the strip's own last row are rows the next strip reads anyway
    const int in_rows_ok = g.H - iy0;
    const unsigned in_row_bytes = (unsigned)(g.W * 8);
    for (int rb = 0; rb < nrows; rb += U) {
        if (rb + U <= nrows && (rb + U) * S + S - 1 + RING < in_rows_ok) {
            unsigned s_ld = s_in + (unsigned)(iy0 + (rb + 1) * S + RING) * in_row_bytes;
            unsigned s_st = s_out + (unsigned)(oy0 + rb) * row_bytes;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                row_mfma((u + 1) % U, nxt);
#pragma unroll
                for (int k = 0; k < S; ++k) {
                    v4i& f = frag[((u + 1) * S + k) % RING];
                    if constexpr (ODDW) {
                        const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)v_in, (int)s_ld, 0));
                        const v2i hi = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)v_in2, (int)s_ld, 0));
                        f = v4i{lo[0], lo[1], hi[0], hi[1]};
                    } else {
                        f = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)v_in, (int)s_ld, 0));
                    }
                    s_ld += in_row_bytes;
                }
                epilogue_store(v_out, s_st, true);
                s_st += row_bytes;
#pragma unroll
                for (int t = 0; t < T; ++t) cur[t] = nxt[t];
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int r = rb + u;  // output row of the strip whose epilogue runs now
                if (r >= nrows) return;  // wave-uniform
                // row r+1: its input rows start (r+1)*S rows into the strip; the ring phase repeats every U rows
                row_mfma((u + 1) % U, nxt);
#pragma unroll
                for (int k = 0; k < S; ++k) frag[((u + 1) * S + k) % RING] = load_row((r + 1) * S + k + RING);
                epilogue_store(v_out, s_out + (unsigned)(oy0 + r) * row_bytes, true);
#pragma unroll
                for (int t = 0; t < T; ++t) cur[t] = nxt[t];
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// The same layer straight from an fp32 blob: quantize_to_int8 (Tensor/ConvolutionLayer.cpp:770-775,
// Tensor/QuantizeX86.cpp:402-490) and the depthwise convolution in ONE launch, for a Float8 input ([N][C/8][H*W][8
// floats]) of at most 128 columns. As two launches the int8 copy of the blob is written and read back (c1: 103 MB in +
// 26 MB out + 26 MB back in + 26 MB out); here every fp32 value is read once and nothing but the result is written.
//
// A wave owns one channel octet x the full width x a strip of output rows and walks along the input rows. A row of the
// blob is W x 32 contiguous bytes; lane l of load k takes bytes 16 (64 k + l) .. + 15 of it -- half a pixel, four
// channels -- so that one load instruction reads 1 KB of whole cache lines (NL = 1..4 loads per row for up to 128
// columns). Loading a whole pixel per lane instead (two 16-byte loads 32 bytes apart) touches every cache line twice,
// and the texture addresser, which works per cache line touched, then bounds the kernel: measured 30 us against 24 us.
// The lane quantizes its four values with the layer's input scale and rounding primitive -- every value once -- and
// writes the four bytes into the wave's own ring of four LDS lines [pixel + 2][8 B] (pixels -2, -1 and the ones past
// the row's end are zero: the padding columns). The matrix operand of lane (n, g) for column chunk c -- pixels 64c + 4n -
// 2 + 2g and + 1 -- is then one aligned 16-byte LDS read per kernel row. LDS instructions of one wave execute in order, so
// the wave needs no barrier between its lanes' writes and reads. The loads run four input rows ahead of the
// quantization in a ring of registers; the matrix instructions of a row run under the quantization of the next one, its
// epilogue follows that. Rows outside the image or past the strip read zero through the buffer descriptor.
template <int S, int EPI, int NL>
__global__ void __launch_bounds__(256, 3) conv_dw3x3_f32in_kernel(const float* __restrict__ x, const int8_t* __restrict__ wa,
                                                               void* __restrict__ out, ConvGeom g, Epilogue ep,
                                                               const float* __restrict__ in_scale_p, float in_half,
                                                               int n_strips, int rps, unsigned in_bytes, unsigned out_bytes) {
    constexpr int RL = 4, PF = 4;      // LDS lines / register stages per wave
    constexpr int NCH = (NL + 1) / 2;  // column chunks of 64 pixels (a matrix operand covers 4 x 16 of them)
    const float in_scale = in_scale_p[0];
    constexpr int T = S == 1 ? 2 : 1;  // A sets
    constexpr int PH = 4 / S;          // output pixels per lane column
    constexpr int LINE = (64 * NCH + 8) * 8;
    __shared__ __attribute__((aligned(16))) int8_t lds_all[4][RL][LINE];
    const int C8 = g.C / 8;
    unsigned bx = blockIdx.x, by = blockIdx.y;
    {  // consecutive strips of a plane and consecutive planes on one XCD (see conv_dw3x3_mfma_kernel)
        const unsigned id = by * gridDim.x + bx, total = gridDim.x * gridDim.y, per = total / 8;
        if (id < per * 8) {
            const unsigned w = (id % 8) * per + id / 8;
            bx = w % gridDim.x, by = w / gridDim.x;
        }
    }
    const int o = by % C8, img = by / C8;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int strip = __builtin_amdgcn_readfirstlane(bx * (blockDim.x >> 6) + wave);
    if (strip >= n_strips) return;  // whole wave
    const int lane = threadIdx.x & 63, n = lane & 15, q = lane >> 4;
    int8_t* const lds = &lds_all[wave][0][0];

    // the padding slots of every line: pixels -2, -1 and 32 NL .. 64 NCH + 5 (the row's own pixels from W on are written
    // as zeros with every row)
    for (int i = lane; i < (2 + 64 * NCH + 6 - 32 * NL) * RL; i += 64) {
        constexpr int PADS = 2 + 64 * NCH + 6 - 32 * NL;
        const int line = i / PADS, k = i % PADS;
        const int slot = k < 2 ? k : 32 * NL + k;
        *reinterpret_cast<v2i*>(lds + line * LINE + slot * 8) = v2i{0, 0};
    }

    // ---- input: this lane's 16 bytes of the row in every load ---------------------------------------------------------
    const unsigned HW32 = (unsigned)(g.H * g.W) * 32u;
    const unsigned s_in = (unsigned)(img * C8 + o) * HW32;
    unsigned v_in[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) v_in[k] = 64 * k + lane < 2 * g.W ? (unsigned)(64 * k + lane) * 16u : DW_OOB;
    const __amdgpu_buffer_rsrc_t rin = dw_rsrc(x, in_bytes);
    const int oy0 = strip * rps;
    const int nrows = min(rps, g.OH - oy0);
    const int iy0 = oy0 * S - g.ph;
    const int nq = (nrows - 1) * S + 3;  // input rows this strip reads
    // Odd strips walk UP: a strip and its neighbour below then read the rows they share at the same end of their walks
    // (both last, or both first), i.e. at about the same time, and the second reader finds them in the XCD's L2 instead
    // of fetching them from memory again (the strips of a plane run side by side on one XCD). Walking up only mirrors
    // the row indices: input row j of the walk is row iy0 + nq - 1 - j, output row r of the walk is the strip's row
    // nrows - 1 - r, and kernel row dy meets the line that holds walk row 2 - dy (the weights are loaded mirrored).
    const bool up = (strip & 1) != 0;  // wave-uniform
    auto issue = [&](int j, v4i (&dst)[NL]) {  // j: input row of the walk
        const int iy = up ? iy0 + nq - 1 - j : iy0 + j;
        const bool ok = iy >= 0 && iy < g.H && j < nq;  // wave-uniform
        // (said to the compiler in so many words: it otherwise loops over the lanes' "different" scalar offsets)
        const unsigned s_row = (unsigned)__builtin_amdgcn_readfirstlane((int)(ok ? s_in + (unsigned)(iy * g.W) * 32u : 0u));
#pragma unroll
        for (int k = 0; k < NL; ++k)
            dst[k] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rin, (int)(ok ? v_in[k] : DW_OOB), (int)s_row, 0));
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
    // lane l of load k holds pixel 32 k + l / 2, channels 4 (l & 1) ..: byte (pixel + 2) * 8 + 4 (l & 1) = 16 + 256 k + 4 l
    auto quant_write = [&](int line, const v4i (&src)[NL]) {
#pragma unroll
        for (int k = 0; k < NL; ++k) *reinterpret_cast<int*>(lds + line * LINE + 16 + 256 * k + 4 * lane) = quant4(src[k]);
    };

    v4i a[3][T];  // a[k]: the kernel row that meets the k-th of an output row's three lines
    {
        const v4i* ap = reinterpret_cast<const v4i*>(wa) + (size_t)o * 3 * T * 64 + lane;
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
            for (int t = 0; t < T; ++t) a[k][t] = ap[((up ? 2 - k : k) * T + t) * 64];
    }
    // (requested before any input row: loads return in order, so the wait for these in front of the first matrix
    // instruction -- which sits inside the loop and is executed on every pass -- then never reaches past a row's loads)
    __builtin_amdgcn_sched_barrier(0);

    v4i ld[PF][NL];
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(j, ld[j]);

    // ---- epilogue constants (as in conv_dw3x3_mfma_kernel) -----------------------------------------------------------
    const int ch = 8 * o + (S == 1 ? 0 : 4 * (q & 1));
    v4i si[T], bi[T], so[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        si[t] = *reinterpret_cast<const v4i*>(ep.scale_in + ch + 4 * t);
        bi[t] = *reinterpret_cast<const v4i*>(ep.bias + ch + 4 * t);
        so[t] = v4i{0, 0, 0, 0};
        if constexpr (EPI != EPI_F32_P4 && EPI != EPI_F32_P8) so[t] = *reinterpret_cast<const v4i*>(ep.scale_out + ch + 4 * t);
    }
    unsigned qh[T][2] = {};
    if constexpr (EPI == EPI_I8_P8_NONNEG) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
            qh[t][0] = dw_clamp_pair(ep, so[t][0], so[t][1]);
            qh[t][1] = dw_clamp_pair(ep, so[t][2], so[t][3]);
        }
    }
    // ---- output: this lane's pixel of the row in every column chunk --------------------------------------------------
    const unsigned OHW = (unsigned)(g.OH * g.OW);
    unsigned v_out[NCH], s_out, row_bytes;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int ox = PH * (16 * c + n) + (S == 1 ? q : (q >> 1));
        const bool st_ok = ox < g.OW;
        if constexpr (EPI == EPI_F32_P4)
            v_out[c] = st_ok ? (S == 1 ? 0u : (unsigned)(q & 1)) * OHW * 16u + (unsigned)ox * 16u : DW_OOB;
        else if constexpr (EPI == EPI_F32_P8)
            v_out[c] = st_ok ? (unsigned)ox * 32u + (S == 1 ? 0u : (unsigned)(q & 1) * 16u) : DW_OOB;
        else
            v_out[c] = st_ok ? (unsigned)ox * 8u + (S == 1 ? 0u : (unsigned)(q & 1) * 4u) : DW_OOB;
    }
    if constexpr (EPI == EPI_F32_P4) s_out = (unsigned)(img * (g.C / 4) + 2 * o) * OHW * 16u, row_bytes = (unsigned)g.OW * 16u;
    else if constexpr (EPI == EPI_F32_P8) s_out = (unsigned)(img * C8 + o) * OHW * 32u, row_bytes = (unsigned)g.OW * 32u;
    else s_out = (unsigned)(img * C8 + o) * OHW * 8u, row_bytes = (unsigned)g.OW * 8u;
    const __amdgpu_buffer_rsrc_t rout = dw_rsrc(out, out_bytes);

    v4i cur[NCH][T];
    auto epilogue_store = [&](int r) {  // output row r of the walk, from cur
        const unsigned s_row =
            (unsigned)__builtin_amdgcn_readfirstlane((int)(s_out + (unsigned)(oy0 + (up ? nrows - 1 - r : r)) * row_bytes));
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if constexpr (EPI == EPI_F32_P4 || EPI == EPI_F32_P8) {
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    const v4i res = dw_dequant4(ep, cur[c][t], si[t], bi[t]);
                    const unsigned vo_t = (t == 0 || v_out[c] == DW_OOB) ? v_out[c] : v_out[c] + (EPI == EPI_F32_P4 ? OHW * 16u : 16u);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_store, res), rout, (int)vo_t, (int)s_row, 0);
                }
            } else {
                constexpr bool NONNEG = EPI == EPI_I8_P8_NONNEG;
                if constexpr (S == 1) {
                    v2i w2;
                    w2[0] = (int)dw_requant4<NONNEG>(ep, cur[c][0], si[0], bi[0], so[0], qh[0][0], qh[0][1]);
                    w2[1] = (int)dw_requant4<NONNEG>(ep, cur[c][T - 1], si[T - 1], bi[T - 1], so[T - 1], qh[T - 1][0], qh[T - 1][1]);
                    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, w2), rout, (int)v_out[c], (int)s_row, 0);
                } else {
                    const unsigned w1 = dw_requant4<NONNEG>(ep, cur[c][0], si[0], bi[0], so[0], qh[0][0], qh[0][1]);
                    __builtin_amdgcn_raw_buffer_store_b32(w1, rout, (int)v_out[c], (int)s_row, 0);
                }
            }
        }
    };
    auto row_mfma = [&](int line0) {  // the three input rows of an output row sit in lines line0, +1, +2 (mod RL)
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            v4i b[3];
#pragma unroll
            for (int dy = 0; dy < 3; ++dy)
                b[dy] = *reinterpret_cast<const v4i*>(lds + ((line0 + dy) % RL) * LINE + (64 * c + 4 * n + 2 * q) * 8);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                cur[c][t] = v4i{0, 0, 0, 0};
#pragma unroll
                for (int dy = 0; dy < 3; ++dy) cur[c][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[dy][t], b[dy], cur[c][t], 0, 0, 0);
            }
        }
    };

    // Input row j of the walk sits in line and register stage j % 4 and completes output row (j - 2) / S when that is
    // whole. Rows 0..2 (everything up to the first output row) run in front of the loop, so that every pass of the loop
    // issues the same loads and stores on every path: the waits for a row's loads are counted back from the youngest
    // request, and a path with fewer requests would pull them (and with them the loads in flight) closer.
    // (where the rows in front of the loop have no output row to store yet they issue stores that go nowhere -- an
    // out-of-range offset -- so that the count of requests behind a row's loads is the loop's own from the first pass on)
    auto no_store = [&](int i) {  // (a different nowhere each time, or the compiler drops all but the last as dead stores)
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int nowhere = (int)(DW_OOB + 256u * (unsigned)i + 64u * (unsigned)c);
            if constexpr (EPI == EPI_F32_P4 || EPI == EPI_F32_P8) {
#pragma unroll
                for (int t = 0; t < T; ++t)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_store, v4i{0, 0, 0, 0}), rout, nowhere + 16 * t, 0, 0);
            } else if constexpr (S == 1) {
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u_store, v2i{0, 0}), rout, nowhere, 0, 0);
            } else {
                __builtin_amdgcn_raw_buffer_store_b32(0u, rout, nowhere, 0, 0);
            }
        }
    };
    auto input_row = [&](int j, int jj, bool store_prev) {  // jj = j modulo 4; both a compile-time constant at every call
        quant_write(jj % RL, ld[jj % PF]);
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
    // (eight rows per pass: the waits the compiler places in the first rows of a pass reach a row or two further back
    // than the ring needs, so the passes are long)
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

// true when the fused fp32 -> depthwise launch takes this layer and blob (Float8 input; the caller has checked
// dw_mfma_applicable)
bool dw_f32in_applicable(const ConvGeom& g, int in_layout) {
    if (in_layout != OTTER_HIP_F32_P8 || g.kh != 3 || g.kw != 3) return false;
    if (g.W > 128 || g.W < 17 || g.C % 8 != 0) return false;
    if ((size_t)g.N * g.C * g.H * g.W * 4 >= ((size_t)1 << 31)) return false;  // 32-bit buffer offsets
    return (long)g.N * (g.C / 8) <= 65535;
}

hipError_t run_conv_dw_f32in(const float* x, const int8_t* wa, void* out, const ConvGeom& g, const Epilogue& ep, int epi,
                             const float* in_scale, int in_round_mode, int strip_rows, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const int C8 = g.C / 8;
    const long planes = (long)g.N * C8;
    if (planes > 65535) return hipErrorInvalidValue;
    // strips of equal height, about two waves per SIMD over the chip (as in run_conv_dw_mfma)
    int rps;
    if (strip_rows > 0) {
        rps = std::min(strip_rows, g.OH);
    } else {
        int ns = 1;
        while (ns < g.OH && ns * planes < 2048) ++ns;
        rps = (g.OH + ns - 1) / ns;
    }
    const int n_strips = (g.OH + rps - 1) / rps;
    const int wpb = n_strips % 4 == 0 ? 4 : (n_strips % 2 == 0 ? 2 : 1);
    const dim3 grid((unsigned)(n_strips / wpb), (unsigned)planes), block(64 * wpb);
    const float in_half = in_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
    // A grid of a few workgroups per CU is resident all at once, and the dispatcher is free to give one CU three of them
    // and another one: the kernel then lasts as long as the fullest CU. Reserving a share of the CU's 160 KB of LDS per
    // workgroup (beyond the 17 KB of lines the kernel uses) caps the workgroups per CU at the even share.
    const long wgs = (long)grid.x * grid.y, per_cu = (wgs + 255) / 256;
    unsigned lds_reserve = 0;
    if (wpb == 4 && per_cu >= 2 && per_cu <= 3) lds_reserve = (unsigned)(160 * 1024 / per_cu - 18 * 1024) / 1024 * 1024;
    if (lds_reserve > 46 * 1024) lds_reserve = 46 * 1024;  // static + dynamic stay within the default 64 KB limit
    const unsigned in_bytes = (unsigned)((size_t)g.N * g.C * g.H * g.W * 4);
    const unsigned out_bytes = (unsigned)((size_t)g.N * g.K * g.OH * g.OW * (epi == EPI_F32_P4 || epi == EPI_F32_P8 ? 4 : 1));
#define OHIP_DWF_L(S_, E_, L_)                                                                                           \
    hipLaunchKernelGGL((conv_dw3x3_f32in_kernel<S_, E_, L_>), grid, block, lds_reserve, stream, x, wa, out, g, ep, in_scale, in_half, \
                       n_strips, rps, in_bytes, out_bytes)
#define OHIP_DWF_N(S_, E_)                       \
    do {                                         \
        switch ((g.W + 31) / 32) {               \
        case 1: OHIP_DWF_L(S_, E_, 1); break;    \
        case 2: OHIP_DWF_L(S_, E_, 2); break;    \
        case 3: OHIP_DWF_L(S_, E_, 3); break;    \
        default: OHIP_DWF_L(S_, E_, 4); break;   \
        }                                        \
    } while (0)
#define OHIP_DWF_E(S_)                                                  \
    do {                                                                \
        if (epi == EPI_I8_P8_NONNEG) OHIP_DWF_N(S_, EPI_I8_P8_NONNEG);  \
        else if (epi == EPI_I8_P8) OHIP_DWF_N(S_, EPI_I8_P8);           \
        else if (epi == EPI_F32_P8) OHIP_DWF_N(S_, EPI_F32_P8);         \
        else OHIP_DWF_N(S_, EPI_F32_P4);                                \
    } while (0)
    if (g.sh == 1) OHIP_DWF_E(1);
    else OHIP_DWF_E(2);
#undef OHIP_DWF_E
#undef OHIP_DWF_N
#undef OHIP_DWF_L
    return hipGetLastError();
}

// the epilogue code of a depthwise layer: the common rule, plus fp32 output in the depthwise default layout Float8
int dw_mfma_epilogue(const Epilogue& ep, int K) {
    const int epi = pick_epilogue(ep, K);
    const bool clamp_act = ep.act == 0 || ep.act == 1 || ep.act == 3 || (ep.act == 2 && ep.lrelu);
    if (epi == EPI_GENERIC && clamp_act && ep.out_kind == OTTER_HIP_OUT_F32 && ep.out_layout == OTTER_HIP_F32_P8 && K % 8 == 0)
        return EPI_F32_P8;
    return epi;
}

// true when this layer / batch can take the matrix-core kernel (the caller falls back to the vector kernels otherwise)
bool dw_mfma_applicable(const ConvGeom& g, const Epilogue& ep, int epi, bool scale_out_positive) {
    if (epi == EPI_I8_P8_NONNEG && !scale_out_positive) return false;  // the clamp is moved past the output scale
    if (!(g.kh == g.kw && (g.kh == 3 || g.kh == 5) && g.dh == 1 && g.dw == 1 && g.sh == g.sw && (g.sh == 1 || g.sh == 2))) return false;
    if (g.ph > g.kh / 2 || !dw_mfma_window_fits(g.kh, g.sh, g.pw) || g.C % 8 != 0 || g.C != g.K) return false;
    if (epi != EPI_I8_P8 && epi != EPI_I8_P8_NONNEG && epi != EPI_F32_P4 && epi != EPI_F32_P8) return false;
    const size_t in_bytes = (size_t)g.N * g.C * g.H * g.W;
    const size_t out_bytes = (size_t)g.N * g.K * g.OH * g.OW * (epi == EPI_F32_P4 || epi == EPI_F32_P8 ? 4 : 1);
    return in_bytes < ((size_t)1 << 31) && out_bytes < ((size_t)1 << 31);  // 32-bit buffer offsets
}

hipError_t run_conv_dw_mfma(const int8_t* x, const int8_t* wa, void* out, const ConvGeom& g, const Epilogue& ep, int epi,
                            int strip_blocks, hipStream_t stream) {
    if (g.N == 0 || g.OH * g.OW == 0) return hipSuccess;
    const int C8 = g.C / 8;
    const int PH = 4 / g.sh;  // output pixels per lane column
    // lane columns an image row needs
    const int cols = (g.OW + PH - 1) / PH;
    int lpi = 16, ipw = 1, col_chunks = (cols + 15) / 16;
    if (cols <= 8) {  // narrow images side by side in one wave
        lpi = cols;
        ipw = std::min(16 / lpi, g.N);
        col_chunks = 1;
    }
    const long groups = (long)((g.N + ipw - 1) / ipw) * C8;
    if (groups > 65535) return hipErrorInvalidValue;  // grid.y limit; the caller splits the batch
    // strip height: the tallest strips (setup and halo rows amortised over the longest walk) that still give about two
    // waves per SIMD (measured: fewer, longer waves win), all of the same height so that the waves finish together
    const int U = 8 / g.sh;
    const int blocks_total = (g.OH + U - 1) / U;
    int rps;
    if (strip_blocks > 0) {
        rps = std::min(strip_blocks, blocks_total) * U;
    } else {
        int ns = 1;
        while (ns < blocks_total && (long)col_chunks * ns * groups < 2048) ++ns;
        rps = (g.OH + ns - 1) / ns;
    }
    const int n_strips = (g.OH + rps - 1) / rps;
    const int wpb = n_strips % 4 == 0 ? 4 : (n_strips % 2 == 0 ? 2 : 1);
    const dim3 grid((unsigned)(col_chunks * (n_strips / wpb)), (unsigned)groups), block(64 * wpb);
    // A grid of at most a few workgroups per CU is resident all at once, and the dispatcher is free to give one CU
    // three of them and another one: the kernel then lasts as long as the fullest CU. Reserving a share of the CU's
    // 160 KB of LDS per workgroup (the kernel uses none) caps the workgroups per CU at the even share.
    constexpr long kCUs = 256;
    const long wgs = (long)grid.x * grid.y;
    const long per_cu = (wgs + kCUs - 1) / kCUs;
    unsigned lds_reserve = 0;
    if (wpb == 4 && per_cu >= 2 && per_cu <= 4) lds_reserve = (unsigned)(160 * 1024 / per_cu) / 1024 * 1024;
    if (lds_reserve > 64 * 1024) lds_reserve = 64 * 1024;  // the default limit of dynamic LDS; still two per CU
    const unsigned in_bytes = (unsigned)((size_t)g.N * g.C * g.H * g.W);
    const unsigned out_bytes = (unsigned)((size_t)g.N * g.K * g.OH * g.OW * (epi == EPI_F32_P4 || epi == EPI_F32_P8 ? 4 : 1));
#define OHIP_DWM_K(S_, E_, O_)                                                                                         \
    do {                                                                                                               \
        if (g.kh == 3)                                                                                                 \
            hipLaunchKernelGGL((conv_dw3x3_mfma_kernel<S_, E_, O_, 3>), grid, block, lds_reserve, stream, x, wa, out, g, ep, \
                               n_strips, rps, col_chunks, lpi, ipw, in_bytes, out_bytes);                              \
        else                                                                                                           \
            hipLaunchKernelGGL((conv_dw3x3_mfma_kernel<S_, E_, O_, 5>), grid, block, lds_reserve, stream, x, wa, out, g, ep, \
                               n_strips, rps, col_chunks, lpi, ipw, in_bytes, out_bytes);                              \
    } while (0)
#define OHIP_DWM(S_, E_) \
    do {                                                                                                               \
        if (g.W & 1)                                                                                                   \
            OHIP_DWM_K(S_, E_, true);                                                                                  \
        else                                                                                                           \
            OHIP_DWM_K(S_, E_, false);                                                                                 \
    } while (0)
#define OHIP_DWM_E(S_)                                                \
    do {                                                              \
        if (epi == EPI_I8_P8_NONNEG) OHIP_DWM(S_, EPI_I8_P8_NONNEG);  \
        else if (epi == EPI_I8_P8) OHIP_DWM(S_, EPI_I8_P8);           \
        else if (epi == EPI_F32_P8) OHIP_DWM(S_, EPI_F32_P8);         \
        else OHIP_DWM(S_, EPI_F32_P4);                                \
    } while (0)
    if (g.sh == 1) OHIP_DWM_E(1);
    else OHIP_DWM_E(2);
#undef OHIP_DWM_E
#undef OHIP_DWM_K
#undef OHIP_DWM
    return hipGetLastError();
}

}  // namespace ohip
