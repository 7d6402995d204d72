// An inverted-residual block -- 1x1 expand (int8 -> int8), depthwise 3x3 stride 1 pad 1 (int8 -> int8), 1x1 project
// (int8 -> fp32 Float4 [+ shortcut sum] [+ the Byte8 quantization of the result], or int8 -> int8) -- as ONE launch.
//
// Layer by layer the expanded tensor (six times the block's input) is written to memory twice and read twice, and at
// 28x28 and below each of the three launches lasts a few microseconds for a microsecond of traffic. Here a workgroup
// (8 waves) owns a band of output rows of one image and keeps everything between the block's input and its output in
// LDS. The expanded channels are walked in slices of SL (64 or 128); per slice
//   A  expand: the band's input pixels (+ one halo row above and below) x SL channels on the matrix cores, requantized
//      into LDS lines [octet][row][pixel + 2][8 bytes] whose borders (image edge, padding columns) stay zero;
//   B  depthwise: the 3x3 window on the matrix cores with the block-diagonal weight operand of conv_dw_mfma.hip (one
//      instruction per kernel row and channel quad, the B operand one 16-byte LDS read of 2 pixels x 8 channels),
//      requantized into LDS in the order of the project layer's B operand [pixel group][16 channels][pixel][16 bytes];
//   C  project: the slice's SL channels are SL/64 reduction steps into accumulators that stay in registers over all
//      slices;
// and after the last slice the project epilogue (dequantize, clamp, shortcut sum, quantized twin) stores the band.
// Two barriers per slice (A|B, B|C); C of one slice and A of the next run without one.
// Every intermediate value is the one the three layers would have written: same accumulators, same epilogue code.
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v4u_blk __attribute__((__vector_size__(4 * sizeof(unsigned))));

constexpr int BLK_NI8 = 6;   // (channel pair, pixel group) items of the project layer per wave, at most (8 waves)
constexpr int BLK_CGE = 3;   // 64-channel reduction steps of the expand layer, at most (192 input channels)
constexpr int BLK_PAIR_DW = 112;  // LDS dwords of one expand channel pair's constants: scale_in, bias, scale_out (32 each), 16 clamps
constexpr int BLK_OCT_DW = 52;    // LDS dwords of one depthwise octet: 3 x 8 weight words, scale_in, bias, scale_out (8 each), 4 clamps

struct BlockArgs {
    const int8_t *x, *w_exp, *w_prj;
    const int32_t* k1;  // expand layer: [channel pair][BLK_PAIR_DW] constants (block_pack_expand_consts)
    const int32_t* k2;  // depthwise layer: [octet][BLK_OCT_DW] weights and constants (block_pack_dw_consts)
    void* out;
    Epilogue e1, e2, e3;
    int Cin8, cgE, mtE;   // input octets; reduction steps and (padded) 16-row tiles of the expand weights
    int Ce, Ce8;          // expanded channels, octets
    int cgP, mtP, Cout;   // project: reduction steps, (padded) 16-row tiles, output channels
    int H, W, HW;
    int RB, bands;        // output rows per band, bands per image
    int slices;           // slices of SL expanded channels
    int cpr, rpi;         // depthwise: lane columns (of 4 pixels) per row, rows per wave item
    int ER, pitch;        // LDS lines per octet (RB + 2), bytes per line
    int GA, GD;           // 16-pixel groups: the band's input rows, the band's output rows
    int npairsP, itemsP;  // project: channel pairs (32 channels), pairs x GD
    unsigned inv_w;       // ceil(2^20 / W)
    int lds_e, lds_d, lds_c1, lds_c2;  // byte offsets: expanded lines, depthwise results, constants of the two layers
    int lds_c3, lds_r;                 // constants of the project layer, the band's shortcut elements (fp32 result only)
    // The slices of a band dealt to `split` workgroups (grid.z), `spp` consecutive slices each: each adds its slices
    // into accumulators of its own, writes them to `partial` and counts itself in at counters[band of the batch]; the
    // last one to arrive adds the others' up and runs the epilogue.
    int split, spp;
    int* partial;        // [band of the batch][split][item][tile 2][lane 64][4] accumulators
    int partial_bytes;
    unsigned* counters;  // zero before the launch, and again after it
};

// LDS visibility between the phases needs the LDS counter only: the weight loads requested ahead stay in flight
__device__ __forceinline__ void blk_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// EPI3: EPI_F32_P4_FUSED (fp32 Float4, optional residual and twin in e3) or EPI_I8_P8 (signed int8 Byte8)
// SL: expanded channels per slice; NI: project items per wave; CGE: reduction steps of the expand layer (at least cgE);
// WV: waves per workgroup (16 where the registers of a quarter SIMD do, 8 with twice the registers otherwise)
template <bool NONNEG, int EPI3, int SL, int NI, int CGE, int WV>
__global__ void __launch_bounds__(64 * WV) conv_block_kernel(const BlockArgs a) {
    extern __shared__ v4i blk_lds[];
    char* const lds = reinterpret_cast<char*>(blk_lds);
    char* const ldsE = lds + a.lds_e;
    char* const ldsD = lds + a.lds_d;
    const int* const ldsC1 = reinterpret_cast<const int*>(lds + a.lds_c1);
    const int* const ldsC2 = reinterpret_cast<const int*>(lds + a.lds_c2);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 15, q = lane >> 4;
    const int band = blockIdx.x, n = blockIdx.y;
    const int s_begin = blockIdx.z * a.spp, s_end = min(s_begin + a.spp, a.slices);
    // bands of nearly equal height (at most RB rows): band b owns rows [b * H / bands, (b + 1) * H / bands)
    const int r0 = band * a.H / a.bands, rows = (band + 1) * a.H / a.bands - r0;
    const int in_row0 = max(r0 - 1, 0), in_row1 = min(r0 + rows, a.H - 1);
    const int in_pix0 = in_row0 * a.W, in_pixN = (in_row1 + 1) * a.W - in_pix0;
    const int out_pixN = rows * a.W;

    constexpr int npairsE = SL / 32, noct = SL / 8, kqs = SL / 16, KSS = SL / 64;
    constexpr int OPW = noct > WV ? noct / WV : 1;  // octets of a slice per wave (16 over 8 waves: two)
    static_assert(noct % WV == 0 || WV % noct == 0, "the octets of a slice divide evenly over the waves");
    // A: pair of the slice and first pixel group of this wave
    const int prE = wave % npairsE, gaE0 = wave / npairsE;
    constexpr int gaEs = WV / npairsE;

    // the expand weights of a slice: this wave's channel pair, every reduction step
    v4i wA[CGE][2];
    // (every load is issued whatever the shape -- indices past the end are clamped to the last valid one -- so that the
    // wait in front of a weight's first use counts the loads requested after it instead of waiting for all of them)
    auto load_wA = [&](int s) {
        const int pair_abs = min(s * npairsE + prE, (a.Ce - 1) / 32);
        const v4i* wg = reinterpret_cast<const v4i*>(a.w_exp) + (size_t)(2 * pair_abs) * 64 + lane;
#pragma unroll
        for (int cg = 0; cg < CGE; ++cg) {
            const size_t o = (size_t)min(cg, a.cgE - 1) * a.mtE * 64;
            wA[cg][0] = wg[o];
            wA[cg][1] = wg[o + 64];
        }
    };

    // ---- prologue: stage the input as MFMA B operands, the per-channel constants of the three layers, the depthwise
    // weights and the band's shortcut elements; zero the expanded lines (their borders are never written). Every array's
    // first round of loads is requested before any is waited for: one memory latency for the lot. ----------------------
    {
        constexpr int T = 64 * WV;
        const int nX = a.GA * a.cgE * 64;
        const int8_t* xi = a.x + (size_t)n * a.Cin8 * a.HW * 8;
        auto load_x = [&](int i, v2i& lo, v2i& hi) {
            const int l = i & 63, t = i >> 6;
            const int ga = t / a.cgE, cg = t - ga * a.cgE;
            const int pix = ga * 16 + (l & 15), oct = 8 * cg + 2 * (l >> 4);
            lo = hi = v2i{0, 0};
            if (i < nX && pix < in_pixN) {
                const int8_t* s = xi + ((size_t)oct * a.HW + in_pix0 + pix) * 8;
                if (oct < a.Cin8) lo = *reinterpret_cast<const v2i*>(s);
                if (oct + 1 < a.Cin8) hi = *reinterpret_cast<const v2i*>(s + (size_t)a.HW * 8);
            }
        };
        v4i* c1 = reinterpret_cast<v4i*>(lds + a.lds_c1);
        const v4i* g1 = reinterpret_cast<const v4i*>(a.k1);
        const int n1 = ((a.Ce + 31) / 32) * (BLK_PAIR_DW / 4);
        v4i* c2 = reinterpret_cast<v4i*>(lds + a.lds_c2);
        const v4i* g2 = reinterpret_cast<const v4i*>(a.k2);
        const int n2 = a.Ce8 * (BLK_OCT_DW / 4);
        // project (fp32 result): [channel pair][scale_in 32][bias 32] (the arrays are padded to whole pairs), and the
        // band's elements of the shortcut blob as [channel quad][pixel of the band]
        constexpr bool F32 = EPI3 != EPI_I8_P8;
        int* c3 = reinterpret_cast<int*>(lds + a.lds_c3);
        const int n3 = F32 ? a.npairsP * 64 : 0;
        auto load_c3 = [&](int i) {
            const int pr = i >> 6, r = i & 63;
            return __float_as_int(r < 32 ? a.e3.scale_in[32 * pr + r] : a.e3.bias[32 * pr + r - 32]);
        };
        v4i* rl = reinterpret_cast<v4i*>(lds + a.lds_r);
        const bool with_res = F32 && a.e3.residual != nullptr;
        const v4i* rg = reinterpret_cast<const v4i*>(a.e3.residual) + (size_t)n * (a.Cout / 4) * a.HW + r0 * a.W;
        const int n4 = with_res ? (a.Cout / 4) * out_pixN : 0;
        auto load_res = [&](int i) {
            const int c4 = i / out_pixN, px = i - c4 * out_pixN;
            return rg[(size_t)c4 * a.HW + px];
        };
        // first round
        v2i xlo, xhi;
        load_x(tid, xlo, xhi);
        v4i k1v = {0, 0, 0, 0}, k2v = {0, 0, 0, 0}, rv = {0, 0, 0, 0};
        int k3v = 0;
        if (tid < n1) k1v = g1[tid];
        if (tid < n2) k2v = g2[tid];
        if (tid < n3) k3v = load_c3(tid);
        if (tid < n4) rv = load_res(tid);
        load_wA(s_begin);
        const int e16 = noct * a.ER * a.pitch / 16;
        v4i* e = reinterpret_cast<v4i*>(ldsE);
        for (int i = tid; i < e16; i += T) e[i] = v4i{0, 0, 0, 0};
        if (tid < nX) blk_lds[tid] = v4i{xlo[0], xlo[1], xhi[0], xhi[1]};
        if (tid < n1) c1[tid] = k1v;
        if (tid < n2) c2[tid] = k2v;
        if (tid < n3) c3[tid] = k3v;
        if (tid < n4) rl[tid] = rv;
        // the rest
        for (int i = tid + T; i < nX; i += T) {
            load_x(i, xlo, xhi);
            blk_lds[i] = v4i{xlo[0], xlo[1], xhi[0], xhi[1]};
        }
        for (int i = tid + T; i < n1; i += T) c1[i] = g1[i];
#pragma unroll 2
        for (int i = tid + T; i < n2; i += T) c2[i] = g2[i];
        for (int i = tid + T; i < n3; i += T) c3[i] = load_c3(i);
#pragma unroll 2
        for (int i = tid + T; i < n4; i += T) rl[i] = load_res(i);
    }

    // B: lane column -> (row within the item, column chunk); selectors that move a row's tap into the lane's byte of
    // the block-diagonal weight operand (dw_mfma_pack_weights: lane (r, g) holds, for pixel slot e, the tap
    // dx = 2g + e - 1 - r/4 of channel 4t + r%4 at byte 8e + 4t + r%4, zero when dx is outside the window)
    const int row_sub = p / a.cpr, nx = p - row_sub * a.cpr;
    const bool laneB = row_sub < a.rpi;
    const int oxB = 4 * nx + q;
    unsigned selB[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int dx = 2 * q + e - 1 - (p >> 2);
        const unsigned none = 0x0c0c0c0cu;
        selB[e] = (dx >= 0 && dx <= 2) ? (none & ~(0xffu << (8 * (p & 3)))) | ((unsigned)dx << (8 * (p & 3))) : none;
    }
    // the depthwise weight operands: only two of an operand's four dwords ever hold a tap, the others stay zero for the
    // whole kernel; and a zero tuple that every fresh accumulation starts from (kept in registers: the compiler would
    // otherwise write four zeros in front of every first matrix instruction)
    v4i wB[3][2];
#pragma unroll
    for (int dy = 0; dy < 3; ++dy) wB[dy][0] = wB[dy][1] = v4i{0, 0, 0, 0};
    v4i zero4 = {0, 0, 0, 0};
    asm volatile("" : "+v"(zero4));
    // C: accumulators and the weights requested a phase ahead
    v4i acc[NI][2];
#pragma unroll
    for (int i = 0; i < NI; ++i) acc[i][0] = acc[i][1] = v4i{0, 0, 0, 0};
    constexpr bool PFP = NI == 1 || (WV == 8 && NI <= 3);  // the project weights are requested a phase ahead where the registers allow
    v4i wP[NI][KSS][2];
    auto load_wP = [&](int s) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int prP = min(wave + WV * i, a.itemsP - 1) % a.npairsP;
#pragma unroll
            for (int ks = 0; ks < KSS; ++ks) {
                const int cgp = min(s * KSS + ks, a.cgP - 1);
                const v4i* wg = reinterpret_cast<const v4i*>(a.w_prj) + ((size_t)cgp * a.mtP + 2 * prP) * 64 + lane;
                wP[i][ks][0] = wg[0], wP[i][ks][1] = wg[64];
            }
        }
    };
    blk_barrier();

    for (int s = s_begin; s < s_end; ++s) {
        // ================= A: expand =================
        if constexpr (PFP) load_wP(s);
        {
            const int pair_abs = s * npairsE + prE;
            if (32 * pair_abs < a.Ce) {  // wave-uniform
                Epi8 prm;
                {
                    const v4i* c = reinterpret_cast<const v4i*>(ldsC1 + pair_abs * BLK_PAIR_DW);
                    const v4i s0 = c[2 * q], s1 = c[2 * q + 1], b0 = c[8 + 2 * q], b1 = c[9 + 2 * q];
                    const v4i o0 = c[16 + 2 * q], o1 = c[17 + 2 * q], ch = c[24 + q];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        prm.si[e] = __int_as_float(s0[e]), prm.si[4 + e] = __int_as_float(s1[e]);
                        prm.bi[e] = __int_as_float(b0[e]), prm.bi[4 + e] = __int_as_float(b1[e]);
                        prm.so[e] = __int_as_float(o0[e]), prm.so[4 + e] = __int_as_float(o1[e]);
                        prm.qh[e] = (unsigned)ch[e];
                    }
                }
                char* const eo = ldsE + (size_t)((4 * prE + q) * a.ER) * a.pitch;
                for (int ga = gaE0; ga < a.GA; ga += gaEs) {
                    v4i c0, c1;
                    {
                        const v4i b = blk_lds[(ga * a.cgE) * 64 + lane];
                        c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wA[0][0], b, zero4, 0, 0, 0);
                        c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wA[0][1], b, zero4, 0, 0, 0);
                    }
#pragma unroll
                    for (int cg = 1; cg < CGE; ++cg)
                        if (cg < a.cgE) {
                            const v4i b = blk_lds[(ga * a.cgE + cg) * 64 + lane];
                            c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wA[cg][0], b, c0, 0, 0, 0);
                            c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wA[cg][1], b, c1, 0, 0, 0);
                        }
                    const int a8[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
                    const v2i r = epi8_quant_i8p8<NONNEG, 0>(a.e1, prm, a8);
                    const int pix = ga * 16 + p;
                    if (pix < in_pixN) {
                        const unsigned ipix = (unsigned)(in_pix0 + pix);
                        const unsigned iy = (ipix * a.inv_w) >> 20;
                        const unsigned ix = ipix - iy * (unsigned)a.W;
                        const int er = (int)iy - (r0 - 1);
                        *reinterpret_cast<v2i*>(eo + er * a.pitch + (ix + 2) * 8) = r;
                    }
                }
            }
        }
        blk_barrier();
        // ================= B: depthwise =================
        if (s + 1 < s_end) load_wA(s + 1);
        {
            const int nrc = (rows + a.rpi - 1) / a.rpi;
#pragma unroll
            for (int k = 0; k < OPW; ++k) {
            const int ol = wave % noct + WV * k;
            const int oct_abs = s * noct + ol;
            if (oct_abs < a.Ce8) {  // wave-uniform
                const int* const c = ldsC2 + oct_abs * BLK_OCT_DW;
#pragma unroll
                for (int dy = 0; dy < 3; ++dy) {
                    const unsigned w0 = (unsigned)c[dy * 8 + (p & 3)], w1 = (unsigned)c[dy * 8 + 4 + (p & 3)];
                    wB[dy][0][0] = (int)__builtin_amdgcn_perm(0u, w0, selB[0]), wB[dy][0][2] = (int)__builtin_amdgcn_perm(0u, w0, selB[1]);
                    wB[dy][1][1] = (int)__builtin_amdgcn_perm(0u, w1, selB[0]), wB[dy][1][3] = (int)__builtin_amdgcn_perm(0u, w1, selB[1]);
                }
                Epi8 prm;
                {
                    const v4i* cv = reinterpret_cast<const v4i*>(c + 24);
                    const v4i s0 = cv[0], s1 = cv[1], b0 = cv[2], b1 = cv[3], o0 = cv[4], o1 = cv[5], ch = cv[6];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        prm.si[e] = __int_as_float(s0[e]), prm.si[4 + e] = __int_as_float(s1[e]);
                        prm.bi[e] = __int_as_float(b0[e]), prm.bi[4 + e] = __int_as_float(b1[e]);
                        prm.so[e] = __int_as_float(o0[e]), prm.so[4 + e] = __int_as_float(o1[e]);
                        prm.qh[e] = (unsigned)ch[e];
                    }
                }
                const char* const ei = ldsE + (size_t)(ol * a.ER) * a.pitch + (4 * nx + 2 * q) * 8;
                char* const dout = ldsD + (size_t)(ol >> 1) * 256 + (ol & 1) * 8;
                for (int rc = WV > noct ? wave / noct : 0; rc < nrc; rc += WV > noct ? WV / noct : 1) {
                    const int orow = rc * a.rpi + row_sub;
                    const int orc = min(orow, a.RB - 1);
                    v4i c0 = zero4, c1 = zero4;
#pragma unroll
                    for (int dy = 0; dy < 3; ++dy) {
                        const v4i b = *reinterpret_cast<const v4i*>(ei + (orc + dy) * a.pitch);
                        c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wB[dy][0], b, dy ? c0 : zero4, 0, 0, 0);
                        c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wB[dy][1], b, dy ? c1 : zero4, 0, 0, 0);
                    }
                    const int a8[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
                    const v2i r = epi8_quant_i8p8<NONNEG, 0>(a.e2, prm, a8);
                    if (laneB && orow < rows && oxB < a.W) {
                        const int pix = orow * a.W + oxB;
                        *reinterpret_cast<v2i*>(dout + (size_t)((pix >> 4) * kqs) * 256 + (pix & 15) * 16) = r;
                    }
                }
            }
            }
        }
        blk_barrier();
        // ================= C: project =================
        if constexpr (!PFP) load_wP(s);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int it = wave + WV * i;
            if (it < a.itemsP) {  // wave-uniform
                const int gd = it / a.npairsP;
#pragma unroll
                for (int ks = 0; ks < KSS; ++ks) {
                    if (s * KSS + ks < a.cgP) {
                        const v4i b = *reinterpret_cast<const v4i*>(ldsD + (size_t)((gd * kqs + 4 * ks + q) * 16 + p) * 16);
                        acc[i][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wP[i][ks][0], b, acc[i][0], 0, 0, 0);
                        acc[i][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wP[i][ks][1], b, acc[i][1], 0, 0, 0);
                    }
                }
            }
        }
    }
    // ---- several workgroups per band: the last to arrive collects the others' accumulators --------------------------
    if (a.split > 1) {
        const int bi = n * a.bands + band;
        // The accumulators travel through memory at agent scope (sc1): the stores go through to the level all compute
        // units share and the loads do not hit in a cache that could hold older data, so the hand-over needs no
        // write-back or invalidation of a whole L2.
        constexpr int AGENT = 1 << 4;
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(a.partial, 0, a.partial_bytes, 0x00020000);
        const unsigned mine = ((unsigned)(bi * a.split + (int)blockIdx.z) * (unsigned)a.itemsP) * 2048u + (unsigned)lane * 16u;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int it = wave + WV * i;
            if (it < a.itemsP) {  // wave-uniform
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_blk, acc[i][0]), rp, (int)(mine + (unsigned)it * 2048u), 0, AGENT);
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_blk, acc[i][1]), rp, (int)(mine + (unsigned)it * 2048u + 1024u), 0, AGENT);
            }
        }
        // A barrier does not wait for the memory counter: every wave first waits until its own stores have been
        // acknowledged (vmcnt(0)), and only then does the barrier say that the whole workgroup's partial sums are
        // visible at agent scope. Without the wait the arrival below could be counted while a store is still in flight,
        // and the last workgroup would add whatever the slot held before.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        int* const flag = reinterpret_cast<int*>(ldsD);  // (the depthwise results are not read any more)
        if (tid == 0) {
            const unsigned before = __hip_atomic_fetch_add(a.counters + bi, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool last = before == (unsigned)(a.split - 1);
            if (last) __hip_atomic_store(a.counters + bi, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
            *flag = last ? 1 : 0;
        }
        __syncthreads();
        if (*flag == 0) return;  // whole workgroup
        for (int z = 0; z < a.split; ++z) {
            if (z == (int)blockIdx.z) continue;
            const unsigned theirs = ((unsigned)(bi * a.split + z) * (unsigned)a.itemsP) * 2048u + (unsigned)lane * 16u;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int it = wave + WV * i;
                if (it < a.itemsP) {  // wave-uniform
                    const v4i t0 = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rp, (int)(theirs + (unsigned)it * 2048u), 0, AGENT));
                    const v4i t1 = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rp, (int)(theirs + (unsigned)it * 2048u + 1024u), 0, AGENT));
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][0][e] += t0[e], acc[i][1][e] += t1[e];
                }
            }
        }
    }
    // ---- the project layer's epilogue (fp32: its constants and the band's shortcut elements wait in LDS) --------------
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int it = wave + WV * i;
        if (it >= a.itemsP) break;  // wave-uniform
        const int prP = it % a.npairsP, gd = it / a.npairsP;
        const int ch0 = 32 * prP + 8 * q;
        const int pix = gd * 16 + p;
        if (ch0 >= a.Cout || pix >= out_pixN) continue;
        const int opix = r0 * a.W + pix;
        const int a8[8] = {acc[i][0][0], acc[i][0][1], acc[i][0][2], acc[i][0][3],
                           acc[i][1][0], acc[i][1][1], acc[i][1][2], acc[i][1][3]};
        Epi8 prm;
        if constexpr (EPI3 == EPI_I8_P8) {
            epi8_load<EPI_I8_P8>(prm, a.e3, ch0);
            const v2i r = epi8_quant_i8p8<false, 0>(a.e3, prm, a8);
            *reinterpret_cast<v2i*>((int8_t*)a.out + ((size_t)(n * (a.Cout / 8) + ch0 / 8) * a.HW + opix) * 8) = r;
        } else {
            // epi4_store_f32p4<true, 0> with the shortcut element and the constants read from LDS
            {
                const v4i* c = reinterpret_cast<const v4i*>(lds + a.lds_c3) + prP * 16 + 2 * q;
                const v4i s0 = c[0], s1 = c[1], b0 = c[8], b1 = c[9];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    prm.si[e] = __int_as_float(s0[e]), prm.si[4 + e] = __int_as_float(s1[e]);
                    prm.bi[e] = __int_as_float(b0[e]), prm.bi[4 + e] = __int_as_float(b1[e]);
                }
            }
            const v4i* const rl = reinterpret_cast<const v4i*>(lds + a.lds_r) + (ch0 / 4) * out_pixN + pix;
            const size_t elem = (size_t)n * a.Cout * a.HW + ((size_t)(ch0 / 4) * a.HW + opix) * 4;
            v2i tw = {0, 0};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (h == 1 && ch0 + 4 >= a.Cout) break;
                v4i r, res = {0, 0, 0, 0};
                if (a.e3.residual != nullptr) res = rl[h * out_pixN];  // wave-uniform
                unsigned qv = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = __fmaf_rn((float)a8[4 * h + e], prm.si[4 * h + e], prm.bi[4 * h + e]);
                    v = fminf(fmaxf(v, a.e3.act_lo), a.e3.act_hi);
                    if (a.e3.residual != nullptr) v = __fadd_rn(v, __int_as_float(res[e]));
                    if (a.e3.twin != nullptr) {  // wave-uniform
                        const float t = __fmul_rn(v, a.e3.twin_scale);
                        const int k = (int)__fadd_rn(t, __builtin_copysignf(a.e3.twin_half, t));
                        qv |= (unsigned)(min(max(k, -127), 127) & 0xff) << (8 * e);
                    }
                    r[e] = __float_as_int(v);
                }
                *reinterpret_cast<v4i*>((float*)a.out + elem + (size_t)h * a.HW * 4) = r;
                tw[h] = (int)qv;
            }
            if (a.e3.twin != nullptr)  // Cout % 8 == 0 then
                *reinterpret_cast<v2i*>(a.e3.twin + ((size_t)(n * (a.Cout / 8) + ch0 / 8) * a.HW + opix) * 8) = tw;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------------------------

// plan[0] = rows per band, plan[1] = bands, plan[2] = slice (expanded channels), plan[3] = LDS bytes, plan[4] = workgroups
// per band (each takes a share of the slices), plan[5] = ints of workspace for their accumulators (0 when plan[4] == 1)
// force_rb / force_sl / force_split: 0 = automatic
bool conv_block_plan(const ConvGeom& ge, const ConvGeom& gp, int force_rb, int force_sl, int force_split, int plan[6],
                     BlockArgs* out) {
    const int W = ge.W, H = ge.H, Ce = ge.K, Cout = gp.K;
    if (W > 64 || W < 1 || H < 1) return false;
    const int cpr = (W + 3) / 4, rpi = 16 / cpr;
    const int cgE = igemm_channel_groups(ge.C);
    if (cgE > BLK_CGE) return false;
    const int npairsP = (Cout + 31) / 32;
    const int pitch = (4 * cpr + 4) * 8;
    constexpr int kLdsMax = 160 * 1024;
    int off[6];  // expanded lines, depthwise results, expand / depthwise / project constants, shortcut elements
    auto fits = [&](int RB, int SL, int* total) {
        const int rows_in = std::min(RB + 2, H);
        const int GA = (rows_in * W + 15) / 16, GD = (RB * W + 15) / 16;
        if (npairsP * GD > 8 * BLK_NI8) return false;
        const int x = GA * cgE * 1024;
        const int e = (SL / 8) * (RB + 2) * pitch;
        const int d = GD * (SL / 16) * 256;
        const int c1 = ((Ce + 31) / 32) * BLK_PAIR_DW * 4, c2 = (Ce / 8) * BLK_OCT_DW * 4;
        off[0] = x, off[1] = off[0] + (e + 255) / 256 * 256, off[2] = off[1] + d, off[3] = off[2] + c1;
        off[4] = off[3] + c2, off[5] = off[4] + npairsP * 256;
        *total = off[5] + (Cout / 4) * RB * W * 16;
        return *total <= kLdsMax;
    };
    int RB = 0, SL = 0, tot = 0;
    bool fill = false;  // bands lowered for the project layer's sake: deal their slices out until the compute units have work
    if (force_rb > 0 || force_sl > 0) {
        RB = force_rb > 0 ? std::min(force_rb, H) : std::min(H, std::max(rpi, 4));
        SL = force_sl == 64 || force_sl == 128 ? force_sl : 64;
        if (!fits(RB, SL, &tot)) return false;
    } else {
        // the tallest band that still gives every compute unit a workgroup (fewer halo rows to expand twice), in steps
        // of the depthwise item's rows; the wider slice where the expanded channels fill it. Two workgroups share a
        // compute unit's LDS where there are more workgroups than compute units.
        // (the narrow slice where the last wide one would be at most half full and is a large share of the work:
        // 192 channels at 28x28 b64 15.2 us as three slices of 64 against 16.4 us as 128 + 64)
        const int sl_first = Ce > 64 && !(Ce < 256 && Ce % 128 != 0 && Ce % 128 <= 64) ? 128 : 64;
        bool found = false;
        for (int rb = (H + rpi - 1) / rpi * rpi; rb >= 1 && !found; rb -= (rb > rpi ? rpi : 1)) {
            const int rbc = std::min(rb, H);
            const long wgs = (long)ge.N * ((H + rbc - 1) / rbc);
            if (wgs < 256 && rbc > std::max(rpi, 4)) continue;
            const int budget = wgs > 256 ? 80 * 1024 : kLdsMax;
            for (int sl = sl_first; sl >= 64 && !found; sl -= 64)
                if (fits(rbc, sl, &tot) && tot <= budget) RB = rbc, SL = sl, found = true;
        }
        if (!found) return false;
        // the bands are of nearly equal height: no taller than the rows divided by their number (28 rows as four bands
        // are bands of 7, not of 8: one pixel group less in every phase, 17.5 -> 16.4 us)
        const int nb = (H + RB - 1) / RB;
        RB = (H + nb - 1) / nb;
        // More than 24 (channel pair, pixel group) tiles of the project layer per band take the kernel variant with six
        // of them per wave, which is slow (7x7 160 -> 960 -> 320 b64: 28 us as one band of 40 tiles dealt to four
        // workgroups, 20.8 us as two bands of 20 dealt to two each): lower bands where that brings the count to 24.
        if (npairsP * ((RB * W + 15) / 16) > 24) {
            for (int rb = RB - 1; rb >= 1; --rb) {
                const int nb2 = (H + rb - 1) / rb, rbt = (H + nb2 - 1) / nb2;
                int t2 = 0;
                if (npairsP * ((rbt * W + 15) / 16) <= 24 && fits(rbt, SL, &t2)) {
                    RB = rbt, fill = true;
                    break;
                }
            }
        }
        fits(RB, SL, &tot);
    }
    plan[0] = RB, plan[1] = (H + RB - 1) / RB, plan[2] = SL, plan[3] = tot;
    // Fewer bands than half the compute units: the slices of a band are dealt to several workgroups
    const int slices = (Ce + SL - 1) / SL;
    const long wgs1 = (long)ge.N * plan[1];
    int split = 1;
    if (force_split > 0) split = force_split;
    else if (wgs1 < 128) split = (int)std::min<long>(slices, 256 / wgs1);
    else if (fill && wgs1 < 256) split = (int)std::min<long>(slices, (256 + wgs1 - 1) / wgs1);  // (at least two per band)
    split = std::max(1, std::min(split, slices));
    const int spp = (slices + split - 1) / split;
    split = (slices + spp - 1) / spp;  // no workgroup without a slice
    const int GDp = (RB * W + 15) / 16;
    plan[4] = split;
    const long ws = split > 1 ? wgs1 * split * npairsP * GDp * 512 : 0;
    if (ws >= (1l << 28) || wgs1 > 65536) return false;
    plan[5] = (int)ws;
    if (out) {
        out->split = split, out->spp = spp;
        BlockArgs& a = *out;
        a.Cin8 = ge.C / 8, a.cgE = cgE, a.mtE = igemm_padded_rows(Ce) / 16;
        a.Ce = Ce, a.Ce8 = Ce / 8;
        a.cgP = igemm_channel_groups(Ce), a.mtP = igemm_padded_rows(Cout) / 16, a.Cout = Cout;
        a.H = H, a.W = W, a.HW = H * W;
        a.RB = RB, a.bands = plan[1], a.slices = (Ce + SL - 1) / SL;
        a.cpr = cpr, a.rpi = rpi, a.ER = RB + 2, a.pitch = pitch;
        a.GA = (std::min(RB + 2, H) * W + 15) / 16, a.GD = (RB * W + 15) / 16;
        a.npairsP = npairsP, a.itemsP = npairsP * a.GD;
        a.inv_w = ((1u << 20) + W - 1) / W;
        a.lds_e = off[0], a.lds_d = off[1], a.lds_c1 = off[2], a.lds_c2 = off[3], a.lds_c3 = off[4], a.lds_r = off[5];
    }
    return true;
}

// the three layers as the kernel needs them: e1 / e2 int8 Byte8 epilogues of one family (both clamp at zero or neither),
// e3 fp32 Float4 (clamp activations) or signed int8 Byte8
bool conv_block_applicable(const ConvGeom& ge, const Epilogue& e1, const ConvGeom& gd, const Epilogue& e2, const ConvGeom& gp,
                           const Epilogue& e3) {
    auto pointwise = [](const ConvGeom& g) {
        return g.groups == 1 && g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.C % 8 == 0;
    };
    if (!pointwise(ge) || !pointwise(gp) || ge.K % 8 || gp.K % 8) return false;
    if (!(gd.groups == gd.C && gd.C == gd.K && gd.kh == 3 && gd.kw == 3 && gd.sh == 1 && gd.sw == 1 && gd.ph == 1 &&
          gd.pw == 1 && gd.dh == 1 && gd.dw == 1))
        return false;
    if (ge.K != gd.C || gd.K != gp.C || ge.H != gd.H || ge.W != gd.W || gd.OH != gp.H || gd.OW != gp.W) return false;
    if (ge.N < 1 || ge.N > 65535) return false;
    if ((size_t)ge.N * std::max(std::max(ge.C, ge.K), gp.K) * ge.H * ge.W * 4 >= (1ull << 32)) return false;
    const int p1 = pick_epilogue(e1, ge.K), p2 = pick_epilogue(e2, gd.K), p3 = pick_epilogue(e3, gp.K);
    if (!((p1 == EPI_I8_P8 || p1 == EPI_I8_P8_NONNEG) && p1 == p2)) return false;
    if (e1.lrelu || e2.lrelu || e3.lrelu || e1.act == 2 || e2.act == 2 || e3.act == 2) return false;
    if (p3 == EPI_I8_P8) return e3.twin == nullptr && e3.residual == nullptr;
    return p3 == EPI_F32_P4;
}

// The per-channel constants of the expand layer as the kernel keeps them in LDS: per pair of 16-row tiles (32 channels)
// [scale_in 32][bias 32][scale_out 32][16 words of two 16-bit upper clamps each]. si / bi / so hold `kpad` (a multiple
// of 32) entries. nonneg: the layer clamps at zero (ReLU / clip) and every output scale is positive.
size_t block_expand_const_bytes(int K) { return (size_t)((K + 31) / 32) * BLK_PAIR_DW * sizeof(int32_t); }
void block_pack_expand_consts(const float* si, const float* bi, const float* so, int K, bool nonneg, float act_hi,
                              float round_half, int32_t* dst) {
    const int pairs = (K + 31) / 32;
    std::vector<unsigned> qh(pairs * 16, 0u);
    if (nonneg) conv_pw_stream_clamps(act_hi, round_half, so, pairs * 32, qh.data());
    for (int pr = 0; pr < pairs; ++pr) {
        int32_t* d = dst + (size_t)pr * BLK_PAIR_DW;
        std::memcpy(d, si + 32 * pr, 128);
        std::memcpy(d + 32, bi + 32 * pr, 128);
        std::memcpy(d + 64, so + 32 * pr, 128);
        std::memcpy(d + 96, qh.data() + 16 * pr, 64);
    }
}

// The depthwise 3x3 layer as the kernel keeps it in LDS: per channel octet [kernel row 3][channel 8] words holding the
// row's three taps in bytes 0..2, then [scale_in 8][bias 8][scale_out 8][4 words of two upper clamps each].
size_t block_dw_const_bytes(int C) { return (size_t)(C / 8) * BLK_OCT_DW * sizeof(int32_t); }
void block_pack_dw_consts(const int8_t* w, const float* si, const float* bi, const float* so, int C, bool nonneg, float act_hi,
                          float round_half, int32_t* dst) {
    std::vector<unsigned> qh(C / 2, 0u);
    if (nonneg) conv_pw_stream_clamps(act_hi, round_half, so, C, qh.data());
    for (int o = 0; o < C / 8; ++o) {
        int32_t* d = dst + (size_t)o * BLK_OCT_DW;
        for (int dy = 0; dy < 3; ++dy)
            for (int c = 0; c < 8; ++c) {
                const int8_t* t = w + (size_t)(8 * o + c) * 9 + dy * 3;
                d[dy * 8 + c] = (int32_t)((uint32_t)(uint8_t)t[0] | (uint32_t)(uint8_t)t[1] << 8 | (uint32_t)(uint8_t)t[2] << 16);
            }
        std::memcpy(d + 24, si + 8 * o, 32);
        std::memcpy(d + 32, bi + 8 * o, 32);
        std::memcpy(d + 40, so + 8 * o, 32);
        std::memcpy(d + 48, qh.data() + 4 * o, 16);
    }
}

// The arrival counters of the bands whose slices are dealt to several workgroups live in static device memory (every
// GPU has its own copy; the address is looked up once per device), in two halves:
//  * launches that run now take the next N x bands words of a ring (the lower half). The last workgroup of a band leaves
//    its word at zero again, so the ring needs no clearing, and launches that overlap on different streams count in
//    different words as long as fewer than BLK_COUNTERS / 2 words are handed out between them;
//  * launches recorded into a HIP graph keep the words they were given for as long as the graph is replayed, so they must
//    never meet the ring: they take theirs from the upper half, which is only handed to captured launches, and a small
//    fill kernel recorded in front of the launch zeroes them on every replay (a replay that was cut short cannot poison
//    the next one). When the upper half has been handed out once it is dealt again from its start: two graphs whose
//    launches share words must then not be replayed at the same time.
constexpr int BLK_COUNTERS = 1 << 17;
static __device__ unsigned blk_counters[BLK_COUNTERS];
static std::mutex g_counter_mutex;
static unsigned* g_counter_ptr[64] = {};
static unsigned g_counter_next[64][2] = {};

__global__ void blk_zero_counters_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

static hipError_t block_counters(int words, hipStream_t stream, unsigned** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    constexpr unsigned HALF = BLK_COUNTERS / 2;
    if (dev < 0 || dev >= 64 || words < 1 || (unsigned)words > HALF) return hipErrorInvalidValue;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if ((e = hipStreamIsCapturing(stream, &cs)) != hipSuccess) return e;
    const int half = cs == hipStreamCaptureStatusNone ? 0 : 1;
    {
        std::lock_guard<std::mutex> lock(g_counter_mutex);
        if (!g_counter_ptr[dev]) {
            void* p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(blk_counters));
            if (e != hipSuccess || !p) return e == hipSuccess ? hipErrorInvalidSymbol : e;
            g_counter_ptr[dev] = static_cast<unsigned*>(p);
        }
        unsigned& next = g_counter_next[dev][half];
        if (next + (unsigned)words > HALF) next = 0;
        *out = g_counter_ptr[dev] + half * HALF + next;
        next += (unsigned)words;
    }
    if (half) {
        hipLaunchKernelGGL(blk_zero_counters_kernel, dim3((words + 255) / 256), dim3(256), 0, stream, *out, words);
        return hipGetLastError();
    }
    return hipSuccess;
}

template <bool NN, int E3, int SL, int NI, int CGE, int WV>
static hipError_t launch_block(const BlockArgs& a, const dim3& grid, size_t lds, hipStream_t stream) {
    // more than the default 64 KB of dynamic LDS has to be asked for, once per kernel and device
    static std::atomic<bool> raised[64] = {};
    if (lds > 64 * 1024) {
        int dev = -1;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (dev < 0 || dev >= 64) return hipErrorInvalidValue;
        if (!raised[dev].load(std::memory_order_acquire)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_block_kernel<NN, E3, SL, NI, CGE, WV>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            raised[dev].store(true, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL((conv_block_kernel<NN, E3, SL, NI, CGE, WV>), grid, dim3(64 * WV), lds, stream, a);
    return hipGetLastError();
}

hipError_t run_conv_block(const int8_t* x, const int8_t* w_exp, const int32_t* k1, const int32_t* k2, const int8_t* w_prj, void* out,
                          const ConvGeom& ge, const Epilogue& e1, const ConvGeom& gd, const Epilogue& e2, const ConvGeom& gp,
                          const Epilogue& e3, int force_rb, int force_sl, int force_split, int* workspace, hipStream_t stream) {
    if (!conv_block_applicable(ge, e1, gd, e2, gp, e3)) return hipErrorInvalidValue;
    BlockArgs a;
    int plan[6];
    if (!conv_block_plan(ge, gp, force_rb, force_sl, force_split, plan, &a)) return hipErrorInvalidValue;
    a.partial = workspace, a.partial_bytes = plan[5] * 4, a.counters = nullptr;
    if (plan[4] > 1) {
        if (!workspace) return hipErrorInvalidValue;
        const hipError_t ce = block_counters(ge.N * plan[1], stream, &a.counters);
        if (ce != hipSuccess) return ce;
    }
    a.x = x, a.w_exp = w_exp, a.k1 = k1, a.k2 = k2, a.w_prj = w_prj, a.out = out;
    a.e1 = e1, a.e2 = e2, a.e3 = e3;
    const dim3 grid((unsigned)a.bands, (unsigned)ge.N, (unsigned)plan[4]);
    const bool nonneg = pick_epilogue(e1, ge.K) == EPI_I8_P8_NONNEG;
    const bool i8 = pick_epilogue(e3, gp.K) == EPI_I8_P8;
    // 16 waves where one reduction step and one project item per wave keep a wave within a quarter of a SIMD's registers;
    // 8 waves, with twice the registers each, for the shapes that would spill there
    const bool wide = plan[2] == 128, w16 = a.cgE == 1 && a.itemsP <= 16, few = a.itemsP <= 24;
#define OHIP_BLK4(NN_, E3_, SL_) \
    (w16 ? launch_block<NN_, E3_, SL_, 1, 1, 16>(a, grid, (size_t)plan[3], stream) \
         : few ? launch_block<NN_, E3_, SL_, 3, BLK_CGE, 8>(a, grid, (size_t)plan[3], stream) \
               : launch_block<NN_, E3_, SL_, BLK_NI8, BLK_CGE, 8>(a, grid, (size_t)plan[3], stream))
#define OHIP_BLK2(NN_, E3_) (wide ? OHIP_BLK4(NN_, E3_, 128) : OHIP_BLK4(NN_, E3_, 64))
    if (nonneg) return i8 ? OHIP_BLK2(true, EPI_I8_P8) : OHIP_BLK2(true, EPI_F32_P4_FUSED);
    return i8 ? OHIP_BLK2(false, EPI_I8_P8) : OHIP_BLK2(false, EPI_F32_P4_FUSED);
#undef OHIP_BLK2
#undef OHIP_BLK4
}

}  // namespace ohip

