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

#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int BLK_WAVES = 8;
constexpr int BLK_NI = 5;    // (channel pair, pixel group) items of the project layer per wave, at most
constexpr int BLK_CGE = 3;   // 64-channel reduction steps of the expand layer, at most (192 input channels)

struct BlockArgs {
    const int8_t *x, *w_exp, *w_dw, *w_prj;
    void* out;
    Epilogue e1, e2, e3;
    int Cin8, cgE, mtE;   // input octets; reduction steps and (padded) 16-row tiles of the expand weights
    int Ce, Ce8;          // expanded channels, octets
    int cgP, mtP, Cout;   // project: reduction steps, (padded) 16-row tiles, output channels
    int H, W, HW;
    int RB, bands;        // output rows per band, bands per image
    int SL, slices;       // expanded channels per slice, slices
    int cpr, rpi;         // depthwise: lane columns (of 4 pixels) per row, rows per wave item
    int ER, pitch;        // LDS lines per octet (RB + 2), bytes per line
    int GA, GD;           // 16-pixel groups: the band's input rows, the band's output rows
    int npairsP, itemsP;  // project: channel pairs (32 channels), pairs x GD
    unsigned inv_w;       // ceil(2^20 / W)
    int lds_e, lds_d;     // byte offsets of the two intermediate arrays (the input operands start at 0)
};

// EPI3: EPI_F32_P4_FUSED (fp32 Float4, optional residual and twin in e3) or EPI_I8_P8 (signed int8 Byte8)
template <bool NONNEG, int EPI3>
__global__ void __launch_bounds__(64 * BLK_WAVES) conv_block_kernel(const BlockArgs a) {
    extern __shared__ v4i blk_lds[];
    char* const lds = reinterpret_cast<char*>(blk_lds);
    char* const ldsE = lds + a.lds_e;
    char* const ldsD = lds + a.lds_d;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 15, q = lane >> 4;
    const int band = blockIdx.x, n = blockIdx.y;
    const int r0 = band * a.RB, rows = min(a.RB, a.H - r0);
    const int in_row0 = max(r0 - 1, 0), in_row1 = min(r0 + rows, a.H - 1);
    const int in_pix0 = in_row0 * a.W, in_pixN = (in_row1 + 1) * a.W - in_pix0;
    const int out_pixN = rows * a.W;

    // ---- prologue: zero the expanded lines (their borders are never written), stage the input as MFMA B operands ----
    {
        const int e16 = (a.SL / 8) * a.ER * a.pitch / 16;
        v4i* e = reinterpret_cast<v4i*>(ldsE);
        for (int i = tid; i < e16; i += 64 * BLK_WAVES) e[i] = v4i{0, 0, 0, 0};
        const int total = a.GA * a.cgE * 64;
        const int8_t* xi = a.x + (size_t)n * a.Cin8 * a.HW * 8;
        for (int i = tid; i < total; i += 64 * BLK_WAVES) {
            const int l = i & 63, t = i >> 6;
            const int ga = t / a.cgE, cg = t - ga * a.cgE;
            const int pix = ga * 16 + (l & 15), oct = 8 * cg + 2 * (l >> 4);
            v2i lo = {0, 0}, hi = {0, 0};
            if (pix < in_pixN) {
                const int8_t* s = xi + ((size_t)oct * a.HW + in_pix0 + pix) * 8;
                if (oct < a.Cin8) lo = *reinterpret_cast<const v2i*>(s);
                if (oct + 1 < a.Cin8) hi = *reinterpret_cast<const v2i*>(s + (size_t)a.HW * 8);
            }
            blk_lds[i] = v4i{lo[0], lo[1], hi[0], hi[1]};
        }
    }

    // ---- lane constants of the three phases ------------------------------------------------------------------------
    const int npairsE = a.SL / 32, noct = a.SL / 8, kqs = a.SL / 16;
    // A: pair of the slice and first pixel group of this wave
    const int prE = wave % npairsE, gaE0 = wave / npairsE, gaEs = BLK_WAVES / npairsE;
    // B: lane column -> (row within the item, column chunk)
    const int row_sub = p / a.cpr, nx = p - row_sub * a.cpr;
    const bool laneB = row_sub < a.rpi;
    const int oxB = 4 * nx + q;
    // C: accumulators
    v4i acc[BLK_NI][2];
#pragma unroll
    for (int i = 0; i < BLK_NI; ++i) acc[i][0] = acc[i][1] = v4i{0, 0, 0, 0};

    __syncthreads();

    for (int s = 0; s < a.slices; ++s) {
        // ================= A: expand =================
        {
            const int pair_abs = s * npairsE + prE;
            if (32 * pair_abs < a.Ce) {  // wave-uniform
                v4i wA[BLK_CGE][2];
                const v4i* wg = reinterpret_cast<const v4i*>(a.w_exp) + (size_t)(2 * pair_abs) * 64 + lane;
#pragma unroll
                for (int cg = 0; cg < BLK_CGE; ++cg)
                    if (cg < a.cgE) {
                        wA[cg][0] = wg[(size_t)cg * a.mtE * 64];
                        wA[cg][1] = wg[(size_t)cg * a.mtE * 64 + 64];
                    }
                Epi8 prm;
                epi8_load<NONNEG ? EPI_I8_P8_NONNEG : EPI_I8_P8>(prm, a.e1, 32 * pair_abs + 8 * q);
                char* const eo = ldsE + (size_t)((4 * prE + q) * a.ER) * a.pitch;
                for (int ga = gaE0; ga < a.GA; ga += gaEs) {
                    v4i c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
#pragma unroll
                    for (int cg = 0; cg < BLK_CGE; ++cg)
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
        __syncthreads();
        // ================= B: depthwise =================
        {
            const int nrc = (rows + a.rpi - 1) / a.rpi;
            for (int ol = wave; ol < noct; ol += BLK_WAVES) {
                const int oct_abs = s * noct + ol;
                if (oct_abs >= a.Ce8) break;  // wave-uniform
                v4i wB[3][2];
                const v4i* wg = reinterpret_cast<const v4i*>(a.w_dw) + (size_t)oct_abs * 6 * 64 + lane;
#pragma unroll
                for (int dy = 0; dy < 3; ++dy)
#pragma unroll
                    for (int t = 0; t < 2; ++t) wB[dy][t] = wg[(dy * 2 + t) * 64];
                Epi8 prm;
                epi8_load<NONNEG ? EPI_I8_P8_NONNEG : EPI_I8_P8>(prm, a.e2, 8 * oct_abs);
                const char* const ei = ldsE + (size_t)(ol * a.ER) * a.pitch + (4 * nx + 2 * q) * 8;
                char* const dout = ldsD + (size_t)(ol >> 1) * 256 + (ol & 1) * 8;
                for (int rc = 0; rc < nrc; ++rc) {
                    const int orow = rc * a.rpi + row_sub;
                    const int orc = min(orow, a.RB - 1);
                    v4i c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
#pragma unroll
                    for (int dy = 0; dy < 3; ++dy) {
                        const v4i b = *reinterpret_cast<const v4i*>(ei + (orc + dy) * a.pitch);
                        c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wB[dy][0], b, c0, 0, 0, 0);
                        c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wB[dy][1], b, c1, 0, 0, 0);
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
        __syncthreads();
        // ================= C: project =================
        {
            const int kss = a.SL / 64;
#pragma unroll
            for (int i = 0; i < BLK_NI; ++i) {
                const int it = wave + BLK_WAVES * i;
                if (it < a.itemsP) {  // wave-uniform
                    const int prP = it % a.npairsP, gd = it / a.npairsP;
                    for (int ks = 0; ks < kss; ++ks) {
                        const int cgp = s * kss + ks;
                        if (cgp >= a.cgP) break;
                        const v4i* wg = reinterpret_cast<const v4i*>(a.w_prj) + ((size_t)cgp * a.mtP + 2 * prP) * 64 + lane;
                        const v4i w0 = wg[0], w1 = wg[64];
                        const v4i b = *reinterpret_cast<const v4i*>(ldsD + (size_t)((gd * kqs + 4 * ks + q) * 16 + p) * 16);
                        acc[i][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, b, acc[i][0], 0, 0, 0);
                        acc[i][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, b, acc[i][1], 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- the project layer's epilogue ------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < BLK_NI; ++i) {
        const int it = wave + BLK_WAVES * i;
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
            epi8_load<EPI_F32_P4>(prm, a.e3, ch0);
            const size_t img = (size_t)n * a.Cout * a.HW;  // floats
            const size_t elem = img + ((size_t)(ch0 / 4) * a.HW + opix) * 4;
            v2i tw = {0, 0};
            tw[0] = (int)epi4_store_f32p4<true, 0>((float*)a.out, a.e3, prm.si, prm.bi, elem, a8[0], a8[1], a8[2], a8[3]);
            if (ch0 + 4 < a.Cout)
                tw[1] = (int)epi4_store_f32p4<true, 0>((float*)a.out, a.e3, prm.si + 4, prm.bi + 4, elem + (size_t)a.HW * 4,
                                                       a8[4], a8[5], a8[6], a8[7]);
            if (a.e3.twin != nullptr)  // Cout % 8 == 0 then
                *reinterpret_cast<v2i*>(a.e3.twin + ((size_t)(n * (a.Cout / 8) + ch0 / 8) * a.HW + opix) * 8) = tw;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------------------------

// plan[0] = rows per band, plan[1] = bands, plan[2] = slice (expanded channels), plan[3] = LDS bytes
// force_rb / force_sl: 0 = automatic
bool conv_block_plan(const ConvGeom& ge, const ConvGeom& gp, int force_rb, int force_sl, int plan[4], BlockArgs* out) {
    const int W = ge.W, H = ge.H, Ce = ge.K, Cout = gp.K;
    if (W > 64 || W < 1 || H < 1) return false;
    const int cpr = (W + 3) / 4, rpi = 16 / cpr;
    const int cgE = igemm_channel_groups(ge.C);
    if (cgE > BLK_CGE) return false;
    const int npairsP = (Cout + 31) / 32;
    const int pitch = (4 * cpr + 4) * 8;
    constexpr int kLdsMax = 64 * 1024;
    auto fits = [&](int RB, int SL, int* lds_e, int* lds_d, int* total) {
        const int rows_in = std::min(RB + 2, H);
        const int GA = (rows_in * W + 15) / 16, GD = (RB * W + 15) / 16;
        if (npairsP * GD > BLK_WAVES * BLK_NI) return false;
        const int x = GA * cgE * 1024;
        const int e = (SL / 8) * (RB + 2) * pitch;
        const int d = GD * (SL / 16) * 256;
        *lds_e = x, *lds_d = x + (e + 255) / 256 * 256, *total = *lds_d + d;
        return *total <= kLdsMax;
    };
    int RB = 0, SL = 0, le = 0, ld = 0, tot = 0;
    if (force_rb > 0 || force_sl > 0) {
        RB = force_rb > 0 ? std::min(force_rb, H) : std::min(H, std::max(rpi, 4));
        SL = force_sl == 64 || force_sl == 128 ? force_sl : 64;
        if (!fits(RB, SL, &le, &ld, &tot)) return false;
    } else {
        // the tallest band that still gives every compute unit a workgroup (fewer halo rows to expand twice), in steps
        // of the depthwise item's rows; the wider slice where the expanded channels fill it and LDS allows
        const int sl_first = Ce > 64 ? 128 : 64;
        bool found = false;
        for (int rb = (H + rpi - 1) / rpi * rpi; rb >= 1 && !found; rb -= (rb > rpi ? rpi : 1)) {
            const int rbc = std::min(rb, H);
            const long wgs = (long)ge.N * ((H + rbc - 1) / rbc);
            if (wgs < 256 && rbc > std::max(rpi, 4)) continue;
            for (int sl = sl_first; sl >= 64 && !found; sl -= 64)
                if (fits(rbc, sl, &le, &ld, &tot)) RB = rbc, SL = sl, found = true;
        }
        if (!found) return false;
    }
    plan[0] = RB, plan[1] = (H + RB - 1) / RB, plan[2] = SL, plan[3] = tot;
    if (out) {
        BlockArgs& a = *out;
        a.Cin8 = ge.C / 8, a.cgE = cgE, a.mtE = igemm_padded_rows(Ce) / 16;
        a.Ce = Ce, a.Ce8 = Ce / 8;
        a.cgP = igemm_channel_groups(Ce), a.mtP = igemm_padded_rows(Cout) / 16, a.Cout = Cout;
        a.H = H, a.W = W, a.HW = H * W;
        a.RB = RB, a.bands = plan[1], a.SL = SL, a.slices = (Ce + SL - 1) / SL;
        a.cpr = cpr, a.rpi = rpi, a.ER = RB + 2, a.pitch = pitch;
        a.GA = (std::min(RB + 2, H) * W + 15) / 16, a.GD = (RB * W + 15) / 16;
        a.npairsP = npairsP, a.itemsP = npairsP * a.GD;
        a.inv_w = ((1u << 20) + W - 1) / W;
        a.lds_e = le, a.lds_d = ld;
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

hipError_t run_conv_block(const int8_t* x, const int8_t* w_exp, const int8_t* w_dw, const int8_t* w_prj, void* out,
                          const ConvGeom& ge, const Epilogue& e1, const ConvGeom& gd, const Epilogue& e2, const ConvGeom& gp,
                          const Epilogue& e3, int force_rb, int force_sl, hipStream_t stream) {
    if (!conv_block_applicable(ge, e1, gd, e2, gp, e3)) return hipErrorInvalidValue;
    BlockArgs a;
    int plan[4];
    if (!conv_block_plan(ge, gp, force_rb, force_sl, plan, &a)) return hipErrorInvalidValue;
    a.x = x, a.w_exp = w_exp, a.w_dw = w_dw, a.w_prj = w_prj, a.out = out;
    a.e1 = e1, a.e2 = e2, a.e3 = e3;
    const dim3 grid((unsigned)a.bands, (unsigned)ge.N), block(64 * BLK_WAVES);
    const bool nonneg = pick_epilogue(e1, ge.K) == EPI_I8_P8_NONNEG;
    const bool i8 = pick_epilogue(e3, gp.K) == EPI_I8_P8;
#define OHIP_BLK(NN_, E3_) hipLaunchKernelGGL((conv_block_kernel<NN_, E3_>), grid, block, (size_t)plan[3], stream, a)
    if (nonneg && i8) OHIP_BLK(true, EPI_I8_P8);
    else if (nonneg) OHIP_BLK(true, EPI_F32_P4_FUSED);
    else if (i8) OHIP_BLK(false, EPI_I8_P8);
    else OHIP_BLK(false, EPI_F32_P4_FUSED);
#undef OHIP_BLK
    return hipGetLastError();
}

}  // namespace ohip
