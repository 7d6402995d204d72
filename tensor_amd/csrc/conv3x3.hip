// Dense int8 3x3 stride-1 convolution on the gfx950 matrix cores with the input halo resident in LDS.
//
// A workgroup owns a run of PT consecutive output pixels of one image (row-major, so a few whole output rows)
// and a block of output channels. The input rows that run touches (+1 halo row above and below, +2 zero columns
// left and right) are staged into LDS ONCE, as [octet pair][row][octet of the pair][PITCH bytes of 8-byte pixels] -
// image rows as they lie in the Byte8 tensor, on a power-of-two pitch - so every input byte is fetched from memory
// once per workgroup instead of nine times, the nine filter taps are nine shifted views of the same LDS tile at
// compile-time offsets from one address register per fragment, and the main loop has no barrier at all:
//   * staging is done by the LDS-DMA path (buffer_load_dwordx4 ... lds): one instruction moves one image row of one
//     octet, 16 bytes = two pixels per lane, global memory -> LDS without passing through registers. Padding costs
//     nothing: lanes on the zero columns and rows outside the image carry an out-of-range buffer offset, for which
//     the hardware writes zeros. The transfer for the NEXT tile is issued as soon as the last matrix instruction of
//     this tile has read LDS, so it runs under the epilogue;
//   * the MFMA "B" operand (16 input channels of one pixel) is two ds_read_b64 per lane (the two octets),
//     conflict-free because the 16 lanes of a row group read 16 consecutive pixels = 128 consecutive bytes;
//   * the MFMA "A" operand (weights) is read straight from global memory, already in MFMA lane order
//     (igemm_pack_weights), one coalesced 1 KB read per 16x64 fragment, prefetched two k-chunks ahead. Every
//     workgroup reads the same <= 147 KB of weights, so they stay in L2.
// Rows of up to 252 pixels take 2048-byte lines (two transfers per line; stride 1 and dilation 1 only).
// An odd image width ends on half a pixel pair: the transfer then brings the first pixel of the next row along, and the
// wave that issued it overwrites that pixel with zeros once its transfers have landed, before the barrier.
// The input must stay below 2 GiB (32-bit offsets).
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr unsigned HALO_OOB = 0x80000000u;  // beyond the buffer descriptor: reads as zero

// S = stride (1 or 2), D = dilation (1 or 2; not both 2): the staged rows are (output rows - 1) * S + 2 * D + 1, a
// lane's pixel sits at column ox * S, and the taps are D pixels / D rows apart. Everything else is the same kernel.
// ODDW: the image width is odd (the pixel slot behind a row's last pixel is cleared after every transfer). A template
// parameter because the 7-fragment tile has no register to spare: with the clearing code compiled in, its int8 and
// fp32 instances spill (measured: 64->64 @56x56 batch 64, 17.5 -> 22.5 us); odd widths use at most 6 fragments.
template <int FM, int FN, int WM, int WN, int EPI, int LOGP, int S = 1, int D = 1, bool ODDW = false>
__global__ void __launch_bounds__(256, 2) conv3x3_halo_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk,
                                                           void* __restrict__ out, ConvGeom g, Epilogue ep, int m_tiles16,
                                                           int c_groups, int r_max, int cb, int tiles_per_img, int prm_ofs,
                                                           int total_tiles, unsigned in_bytes, int tile_inv) {
    static_assert(WM * WN == 4 && FM % 2 == 0, "four waves, row fragments in pairs");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int PT = WN * FN * 16;
    constexpr int PITCH = 1 << LOGP;  // bytes per (octet, row) line in LDS; holds pixels -2 .. W+1

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    const int mt_base = blockIdx.y * (WM * FM) + wm * FM;  // first 16-row tile of this wave
    const int OHW = g.OH * g.OW;
    const int C8 = g.C / 8;
    const int EW = g.W + 4;                  // pixels -2 .. W+1 of a row, 8 bytes each (EW * 8 <= PITCH)
    const int pair_bytes = r_max * 2 * PITCH;  // LDS bytes between octet pairs
    // The per-channel epilogue constants of this workgroup's row block go to LDS now (behind the halo tile), so
    // that the epilogue does not end on a chain of global-memory round trips.
    constexpr int ROWS = WM * FM * 16;
    // (a separate LDS object from the halo tile: the compiler then knows that reading it does not touch what the
    // LDS-DMA transfers write, and does not make the epilogue wait for the transfers of the next tile)
    __shared__ __attribute__((aligned(16))) float lds_prm[3 * ROWS];
    for (int i = tid; i < 3 * ROWS; i += 256) {
        const int which = i / ROWS, c = blockIdx.y * ROWS + (i - which * ROWS);
        const float* src = which == 0 ? ep.scale_in : (which == 1 ? ep.bias : ep.scale_out);
        lds_prm[i] = src ? src[c] : 1.f;
    }
    // (int8 result behind ReLU / clip: the upper clamp of the rounded value per channel, once per workgroup instead of
    // once per tile and wave)
    __shared__ __attribute__((aligned(16))) unsigned lds_qh[ROWS / 2];
    if constexpr (EPI == EPI_I8_P8_NONNEG) {
        for (int i = tid; i < ROWS / 2; i += 256) {
            const int c = blockIdx.y * ROWS + 2 * i;
            lds_qh[i] = epi8_clamp_pair(ep, ep.scale_out[c], ep.scale_out[c + 1]);
        }
    }

    const __amdgpu_buffer_rsrc_t rin = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(x), 0, (int)in_bytes, 0x00020000);

    // tile index -> (image, first pixel); consecutive tiles (which share halo rows) go to the same XCD / L2
    auto tile_of = [&](int wg0, int& n, int& p0) {
        int wg = wg0;
        const int per = total_tiles / 8;
        if (per > 0 && wg < per * 8) wg = (wg % 8) * per + wg / 8;
        n = wg / tiles_per_img;
        p0 = (wg % tiles_per_img) * PT;
    };
    // Issue the LDS-DMA transfers of one (tile, channel block): this wave moves octets wave, wave+4, ...
    auto stage = [&](int n, int p0, int cb0) {
        const int p_last = min(p0 + PT, OHW) - 1;
        const int r_lo = p0 / g.OW;
        const int R = (p_last / g.OW - r_lo) * S + 2 * D + 1;
        if constexpr (LOGP == 9) {
            // 512-byte lines: one instruction moves a row of BOTH octets of a pair (adjacent lines in LDS): lanes 0-31
            // the first octet, lanes 32-63 the second, 16 bytes = pixels 2*pp-2 and 2*pp-1 each
            const int hl = lane >> 5, pp = lane & 31;
            const bool col_ok = pp >= 1 && 2 * pp - 2 < g.W;  // (an odd width: the last pair is half padding, see fix_odd)
            const unsigned v_px = (unsigned)(2 * pp - 2) * 8u;
            const unsigned v_both = col_ok ? v_px + (unsigned)hl * (unsigned)(g.H * g.W * 8) : HALO_OOB;
            const unsigned v_first = (col_ok && hl == 0) ? v_px : HALO_OOB;  // an odd octet count ends on half a pair
            if (2 * pp < EW) {
                for (int pj = wave; pj < cb / 16; pj += 4) {
                    const int o = cb0 / 8 + 2 * pj;
                    const bool both = o + 1 < C8;
                    for (int r = 0; r < R; ++r) {
                        const int iy = r_lo * S - g.ph + r;
                        const bool ok = o < C8 && iy >= 0 && iy < g.H;  // wave-uniform
                        const unsigned s_off = ok ? (unsigned)((n * C8 + o) * g.H + iy) * (unsigned)(g.W * 8) : 0u;
                        int8_t* dst = lds + (size_t)pj * pair_bytes + (size_t)((2 * r) << LOGP);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, (__attribute__((address_space(3))) void*)dst, 16,
                                                                 (int)(ok ? (both ? v_both : v_first) : HALO_OOB), (int)s_off,
                                                                 0, 0);
                    }
                }
            }
        } else if constexpr (LOGP == 10) {
            const bool col_ok = lane >= 1 && 2 * lane - 2 < g.W;  // lane: pixels 2*lane-2 and 2*lane-1
            const unsigned v_col = col_ok ? (unsigned)(2 * lane - 2) * 8u : HALO_OOB;
            if (2 * lane < EW) {
                for (int oc = wave; oc < cb / 8; oc += 4) {
                    const int o = cb0 / 8 + oc;
                    for (int r = 0; r < R; ++r) {
                        const int iy = r_lo * S - g.ph + r;
                        const bool ok = o < C8 && iy >= 0 && iy < g.H;  // wave-uniform
                        const unsigned s_off = ok ? (unsigned)((n * C8 + o) * g.H + iy) * (unsigned)(g.W * 8) : 0u;
                        int8_t* dst = lds + (size_t)(oc >> 1) * pair_bytes + (size_t)((2 * r + (oc & 1)) << LOGP);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, (__attribute__((address_space(3))) void*)dst, 16,
                                                                 (int)(ok ? v_col : HALO_OOB), (int)s_off, 0, 0);
                    }
                }
            }
        } else {
            // 2048-byte lines (rows of up to 252 pixels): two transfers per line, 1 KB = 128 pixels each
            constexpr int SEGS = 1 << (LOGP - 10);
            unsigned v_col[SEGS];
            bool seg_on[SEGS];
#pragma unroll
            for (int sg = 0; sg < SEGS; ++sg) {
                const int pl = lane + 64 * sg;  // pixel pair: pixels 2*pl-2 and 2*pl-1
                const bool col_ok = pl >= 1 && 2 * pl - 2 < g.W;
                v_col[sg] = col_ok ? (unsigned)(2 * pl - 2) * 8u : HALO_OOB;
                seg_on[sg] = 2 * pl < EW;
            }
            for (int oc = wave; oc < cb / 8; oc += 4) {
                const int o = cb0 / 8 + oc;
                for (int r = 0; r < R; ++r) {
                    const int iy = r_lo * S - g.ph + r;
                    const bool ok = o < C8 && iy >= 0 && iy < g.H;  // wave-uniform
                    const unsigned s_off = ok ? (unsigned)((n * C8 + o) * g.H + iy) * (unsigned)(g.W * 8) : 0u;
                    int8_t* dst = lds + (size_t)(oc >> 1) * pair_bytes + (size_t)((2 * r + (oc & 1)) << LOGP);
#pragma unroll
                    for (int sg = 0; sg < SEGS; ++sg)
                        if (seg_on[sg])
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, (__attribute__((address_space(3))) void*)(dst + 1024 * sg),
                                                                     16, (int)(ok ? v_col[sg] : HALO_OOB), (int)s_off, 0, 0);
                }
            }
        }
    };

    // Odd width: pixel W (the right zero column, LDS pixel index W + 2) of every line this wave staged holds the next
    // row's first pixel; zero it. Runs after the wave's own transfers have landed and before the barrier, over exactly
    // the (octet, row) lines the loops of stage() give this wave.
    auto fix_odd = [&](int p0) {
        if constexpr (!ODDW) return;
        const int p_last = min(p0 + PT, OHW) - 1;
        const int R = (p_last / g.OW - p0 / g.OW) * S + 2 * D + 1;
        // lane = octet of the stage (at most 64 octets = 512 channels per stage); the wave that staged octet oc: pairs go
        // round the four waves (512-byte lines, both octets of a pair in one transfer), or single octets do
        const int oc = lane;
        const int owner = LOGP == 9 ? (oc >> 1) & 3 : oc & 3;
        if (oc < cb / 8 && owner == wave) {
            int8_t* line = lds + (size_t)(oc >> 1) * pair_bytes + (size_t)((oc & 1) << LOGP) + (g.W + 2) * 8;
            for (int r = 0; r < R; ++r) *reinterpret_cast<v2i*>(line + (size_t)((2 * r) << LOGP)) = v2i{0, 0};
        }
    };

    int n, p0;
    if ((int)blockIdx.x < total_tiles) {
        tile_of(blockIdx.x, n, p0);
        stage(n, p0, 0);
    }

    // Persistent workgroups: the grid holds at most two workgroups per CU and each walks over tiles.
    int bcc[FN];
    for (int wg0 = blockIdx.x; wg0 < total_tiles; wg0 += gridDim.x) {
        tile_of(wg0, n, p0);
        const int r_lo = p0 / g.OW;

        // LDS address of this lane's pixel (tap 0,0) per fragment, octet pair lane/16 of the current k-chunk; walks
        // forward by one chunk after the ninth tap and is wound back at the end of a stage
        // (kept as LDS byte offsets: a generic pointer here would turn the ds_read into a flat load).
        // When every tile is a whole number of image rows and the image a whole number of tiles (no ragged last
        // tile, whose lanes past the image end would keep a clamped pixel) the offsets are the same for every
        // tile: computed once.
        if (wg0 == (int)blockIdx.x || !tile_inv) {
#pragma unroll
            for (int f = 0; f < FN; ++f) {
                const int pix = min(p0 + (wn * FN + f) * 16 + (lane & 15), OHW - 1);
                const int oy = pix / g.OW, ox = pix % g.OW;
                bcc[f] = (oy - r_lo) * S * 2 * PITCH + (ox * S - g.pw + 2) * 8 + (lane >> 4) * pair_bytes;
            }
        }

        v4i acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int f = 0; f < FN; ++f) acc[i][f] = v4i{0, 0, 0, 0};

        const int nck = cb / 64;  // k-chunks per tap in one staged channel block
        const int8_t* wlane = wpk + ((size_t)mt_base * 64 + lane) * 16;
        const size_t kc_stride = (size_t)m_tiles16 * 1024;

        for (int cb0 = 0; cb0 < c_groups * 64; cb0 += cb) {
            // Main loop: no barrier, no branch. The nine taps are unrolled; weight fragments travel through a ring of
            // three register stages and are requested two k-chunks (~0.4 us of MFMA work) before use. Every load is
            // unconditional (the weight rows are padded to whole row blocks and the chunk index is clamped), so that
            // the compiler can count outstanding loads and wait only for the oldest stage.
            constexpr int RD = FN >= 7 ? 2 : 3;  // weight ring depth: the widest tile has registers for two stages only
            v4i ring[RD][FM];
            const int cg0 = cb0 / 64;
            auto a_ptr = [&](int cc, int tap) { return wlane + (size_t)(tap * c_groups + cg0 + cc) * kc_stride; };
            auto load_a = [&](int cc, int tap, v4i (&a)[FM]) {
                const int8_t* p = a_ptr(cc, tap);
#pragma unroll
                for (int i = 0; i < FM; ++i) a[i] = *reinterpret_cast<const v4i*>(p + i * 1024);
            };
            typedef __attribute__((address_space(3))) const int8_t* lds_cptr;
            typedef __attribute__((address_space(3))) const v2i* lds_v2i;
            const lds_cptr lds3 = (lds_cptr)lds;
            auto read_b = [&](int off) {
                const v2i lo = *(lds_v2i)(lds3 + off);
                const v2i hi = *(lds_v2i)(lds3 + off + PITCH);
                return v4i{lo[0], lo[1], hi[0], hi[1]};
            };
            // the halo transfers of this stage were issued one stage ago: wait for this wave's, then for everyone's
            __builtin_amdgcn_s_waitcnt(0);
            fix_odd(p0);
            __syncthreads();
            load_a(0, 0, ring[0]);
            if constexpr (RD == 3) load_a(0, 1, ring[1]);
            v4i b[FN];
#pragma unroll
            for (int f = 0; f < FN; ++f) b[f] = read_b(bcc[f]);
            // The schedule is written out by hand, one group per pixel fragment: the FM matrix instructions that use
            // b[f], then the LDS read that refills b[f] for the NEXT tap (in place: its last reader has just issued),
            // then one weight-fragment load for the tap after next. Every operand is requested several hundred
            // cycles before its use and no extra registers are needed; the barriers pin the order.
            for (int cc = 0; cc < nck; ++cc) {
                const int cc_next = min(cc + 1, nck - 1);
                const int to_next = (cc_next - cc) * 4 * pair_bytes;  // the last chunk re-reads itself: unused data
#pragma unroll
                for (int tap = 0; tap < 9; ++tap) {
                    constexpr int AH = RD - 1;  // taps ahead
                    const int8_t* pa = tap + AH < 9 ? a_ptr(cc, tap + AH) : a_ptr(cc_next, tap + AH - 9);
                    constexpr int kRowB = 2 * PITCH;
                    const int nofs = tap < 8 ? ((tap + 1) / 3) * D * kRowB + ((tap + 1) % 3) * D * 8 : 0;  // compile-time
#pragma unroll
                    for (int f = 0; f < FN; ++f) {
#pragma unroll
                        for (int i = 0; i < FM; ++i)
                            acc[i][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[tap % RD][i], b[f], acc[i][f], 0, 0, 0);
                        if (tap == 8) bcc[f] += to_next;
                        b[f] = read_b(bcc[f] + nofs);
                        if (f < FM) ring[(tap + AH) % RD][f] = *reinterpret_cast<const v4i*>(pa + f * 1024);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if constexpr (RD == 2) {
                    // nine taps flip the parity of a two-stage ring: move the fragments just requested (next chunk,
                    // tap 0) to the stage tap 0 reads
#pragma unroll
                    for (int i = 0; i < FM; ++i) ring[0][i] = ring[1][i];
                }
            }
#pragma unroll
            for (int f = 0; f < FN; ++f) bcc[f] -= (nck - 1) * 4 * pair_bytes;
            // drain the (unused) weight fragments requested past the last tap, so that no register has a load pending
            // when the transfers below are issued: the compiler then needs no memory wait inside the epilogue
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            __syncthreads();  // everyone is done reading this stage: its LDS may be overwritten
            // next stage = next channel block of this tile, or the first block of this workgroup's next tile: its
            // transfers run under the rest of this tile's work (the epilogue, for the last block)
            if (cb0 + cb < c_groups * 64) {
                stage(n, p0, cb0 + cb);
            } else if (wg0 + (int)gridDim.x < total_tiles) {
                int n2, p2;
                tile_of(wg0 + gridDim.x, n2, p2);
                stage(n2, p2, 0);
            }
        }

        // ---- epilogue (no early exits inside the unrolled loops: the accumulators must stay in registers) -------
        const int gq = lane >> 4;
#pragma unroll
        for (int ip = 0; ip < FM / 2; ++ip) {
            const int ch0 = 32 * (mt_base / 2 + ip) + 8 * gq;
            const bool ch_ok = ch0 < g.K;
            Epi8 prm;
            if constexpr (EPI != EPI_GENERIC) {
                // The constants come from LDS through hand-written reads: the compiler would order a ds_read it can
                // see after the LDS-DMA transfers issued above (they write LDS) by waiting for all of them, which
                // would put the next tile's halo transfer back on the critical path. The constants live in their own
                // LDS array, which the transfers never touch.
                const int cl = ch0 - blockIdx.y * ROWS;  // channel within the row block
                const unsigned pa = (unsigned)(size_t)(__attribute__((address_space(3))) float*)lds_prm + (unsigned)cl * 4u;
                v4i r0, r1, r2, r3, r4, r5;
                asm volatile("ds_read_b128 %0, %1" : "=v"(r0) : "v"(pa));
                asm volatile("ds_read_b128 %0, %1 offset:16" : "=v"(r1) : "v"(pa));
                asm volatile("ds_read_b128 %0, %1" : "=v"(r2) : "v"(pa + ROWS * 4));
                asm volatile("ds_read_b128 %0, %1 offset:16" : "=v"(r3) : "v"(pa + ROWS * 4));
                asm volatile("ds_read_b128 %0, %1" : "=v"(r4) : "v"(pa + 2 * ROWS * 4));
                asm volatile("ds_read_b128 %0, %1 offset:16" : "=v"(r5) : "v"(pa + 2 * ROWS * 4));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    prm.si[e] = __int_as_float(r0[e]);
                    prm.si[4 + e] = __int_as_float(r1[e]);
                    prm.bi[e] = __int_as_float(r2[e]);
                    prm.bi[4 + e] = __int_as_float(r3[e]);
                    prm.so[e] = __int_as_float(r4[e]);
                    prm.so[4 + e] = __int_as_float(r5[e]);
                }
                if constexpr (EPI == EPI_I8_P8_NONNEG) {
                    const unsigned pq = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned*)lds_qh + (unsigned)cl * 2u;
                    v4i r6;
                    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(r6) : "v"(pq));
#pragma unroll
                    for (int e = 0; e < 4; ++e) prm.qh[e] = (unsigned)r6[e];
                }
            }
#pragma unroll
            for (int f = 0; f < FN; ++f) {
                const int pix = p0 + (wn * FN + f) * 16 + (lane & 15);
                int a8[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a8[e] = acc[2 * ip][f][e];
                    a8[4 + e] = acc[2 * ip + 1][f][e];
                }
                if (ch_ok && pix < OHW) {
                    if constexpr (EPI == EPI_I8_P8 || EPI == EPI_I8_P8_NONNEG) {
                        epi8_store_i8p8<EPI == EPI_I8_P8_NONNEG>((int8_t*)out, ep, prm,
                                                                 elem_offset(8, n, ch0, pix, g.K, OHW), a8);
                    } else if constexpr (EPI == EPI_F32_P4) {
                        epi4_store_f32p4((float*)out, ep, prm.si, prm.bi, elem_offset(4, n, ch0, pix, g.K, OHW), a8[0],
                                         a8[1], a8[2], a8[3]);
                        if (ch0 + 4 < g.K)
                            epi4_store_f32p4((float*)out, ep, prm.si + 4, prm.bi + 4,
                                             elem_offset(4, n, ch0 + 4, pix, g.K, OHW), a8[4], a8[5], a8[6], a8[7]);
                    } else {
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

namespace {

constexpr int kMaxLdsBytes = 64 * 1024;  // halo tile per workgroup: leaves room for two workgroups per CU (160 KB)
constexpr int kPrmLdsBytes = 3 * 128 * 4 + 16;  // epilogue constants behind it

struct HaloPlan {
    int fn, r_max, cb, tiles_per_img, logp;
    size_t lds_bytes;
    double cost;
};

// input rows a run of pt output pixels starting at a multiple of pt can touch (stride s, dilation d), halo included
int halo_rows(int pt, int OW, int OHW, int s, int d) {
    int worst = 0;
    for (int p0 = 0; p0 < OHW; p0 += pt) {
        const int last = (p0 + pt < OHW ? p0 + pt : OHW) - 1;
        const int rows = (last / OW - p0 / OW) * s + 2 * d + 1;
        if (rows > worst) worst = rows;
    }
    return worst;
}

// The per-lane LDS offsets of a tile may be reused for the workgroup's next tile only if every tile covers the same
// pixels relative to its first row: tiles are whole image rows AND no tile is cut short by the end of the image.
bool halo_tile_invariant(int pt, int OW, int OHW) { return pt % OW == 0 && OHW % pt == 0; }

// grid.y = row blocks of rows_per_wg / 16 sixteen-row tiles; grid.x = persistent workgroups, two resident per CU
void halo_grid(int mpad, int tiles16_per_wg, int total_tiles, int* m_blocks, int* grid_x) {
    *m_blocks = (mpad / 16 + tiles16_per_wg - 1) / tiles16_per_wg;
    int gx = 512 / *m_blocks;
    if (gx < 8) gx = 8;
    if (gx > total_tiles) gx = total_tiles;
    *grid_x = gx;
}

template <int FM, int FN, int WM, int WN, int EPI, int LOGP, int S, int D, bool ODDW>
hipError_t launch_halo_w(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const HaloPlan& pl, hipStream_t stream) {
    auto kern = conv3x3_halo_kernel<FM, FN, WM, WN, EPI, LOGP, S, D, ODDW>;
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kMaxLdsBytes + kPrmLdsBytes);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int mpad = igemm_padded_rows(g.K);
    const int prm_ofs = (int)((pl.lds_bytes + 15) / 16 * 16);
    const int total_tiles = g.N * pl.tiles_per_img;
    int m_blocks, grid_x;
    halo_grid(mpad, WM * FM, total_tiles, &m_blocks, &grid_x);
    const unsigned in_bytes = (unsigned)((size_t)g.N * g.C * g.H * g.W);
    hipLaunchKernelGGL(kern, dim3(grid_x, m_blocks), dim3(256), prm_ofs + 3 * WM * FM * 16 * sizeof(float), stream, x, wpk,
                       out, g, ep, mpad / 16, igemm_channel_groups(g.C), pl.r_max, pl.cb, pl.tiles_per_img, prm_ofs,
                       total_tiles, in_bytes, halo_tile_invariant(WN * FN * 16, g.OW, g.OH * g.OW) ? 1 : 0);
    return hipGetLastError();
}

template <int FM, int FN, int WM, int WN, int EPI, int LOGP, int S, int D>
hipError_t launch_halo_p(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const HaloPlan& pl, hipStream_t stream) {
    if (g.W & 1) {
        if constexpr (FN <= 6) return launch_halo_w<FM, FN, WM, WN, EPI, LOGP, S, D, true>(x, wpk, out, g, ep, pl, stream);
        return hipErrorInvalidValue;  // (the planner gives odd widths at most 6 fragments)
    }
    return launch_halo_w<FM, FN, WM, WN, EPI, LOGP, S, D, false>(x, wpk, out, g, ep, pl, stream);
}

template <int FM, int FN, int WM, int WN, int EPI>
hipError_t launch_halo_e(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const HaloPlan& pl, hipStream_t stream) {
    // the strided and the dilated variant exist for row blocks of 64 channels and more (FM == 4)
    if constexpr (FM == 4) {
        if (g.sh == 2) {
            if (pl.logp == 9) return launch_halo_p<FM, FN, WM, WN, EPI, 9, 2, 1>(x, wpk, out, g, ep, pl, stream);
            return launch_halo_p<FM, FN, WM, WN, EPI, 10, 2, 1>(x, wpk, out, g, ep, pl, stream);
        }
        if (g.dh == 2) {
            if (pl.logp == 9) return launch_halo_p<FM, FN, WM, WN, EPI, 9, 1, 2>(x, wpk, out, g, ep, pl, stream);
            return launch_halo_p<FM, FN, WM, WN, EPI, 10, 1, 2>(x, wpk, out, g, ep, pl, stream);
        }
    }
    if (g.sh != 1 || g.dh != 1) return hipErrorInvalidValue;
    if (pl.logp == 9) return launch_halo_p<FM, FN, WM, WN, EPI, 9, 1, 1>(x, wpk, out, g, ep, pl, stream);
    if (pl.logp == 11) {
        if constexpr (FN <= 6) return launch_halo_p<FM, FN, WM, WN, EPI, 11, 1, 1>(x, wpk, out, g, ep, pl, stream);
        return hipErrorInvalidValue;  // (the planner gives such rows at most 6 fragments)
    }
    return launch_halo_p<FM, FN, WM, WN, EPI, 10, 1, 1>(x, wpk, out, g, ep, pl, stream);
}

template <int FM, int FN, int WM, int WN>
hipError_t launch_halo(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                       const HaloPlan& pl, hipStream_t stream) {
    switch (pick_epilogue(ep, g.K)) {
    case EPI_I8_P8:
        return launch_halo_e<FM, FN, WM, WN, EPI_I8_P8>(x, wpk, out, g, ep, pl, stream);
    case EPI_I8_P8_NONNEG:
        return launch_halo_e<FM, FN, WM, WN, EPI_I8_P8_NONNEG>(x, wpk, out, g, ep, pl, stream);
    case EPI_F32_P4:
        return launch_halo_e<FM, FN, WM, WN, EPI_F32_P4>(x, wpk, out, g, ep, pl, stream);
    default:
        return hipErrorInvalidValue;  // other epilogues take the generic implicit-GEMM kernel
    }
}

// Wave layout: K > 64 -> 2 (channel halves) x 2 (pixel halves), a workgroup covers 128 output channels x 32*FN
// pixels; K <= 64 -> 1 x 4, 64 channels x 64*FN pixels. FM = 4 either way. FN is chosen so that the workgroup
// count fills the 256 CUs x 2 resident workgroups with the least idle tail.
bool plan_halo(const ConvGeom& g, int force_fn, HaloPlan* best) {
    const int OHW = g.OH * g.OW;
    const int cpad = igemm_channel_groups(g.C) * 64;
    const bool wide = igemm_padded_rows(g.K) > 64;
    const int m_blocks = wide ? (igemm_padded_rows(g.K) / 16 + 7) / 8 : 1;
    // LDS line pitch: 512 bytes hold rows of up to 60 pixels (+4 padding pixels), 1024 bytes up to 124, 2048 bytes up to
    // 252 (stride 1, dilation 1 only)
    const int logp = (g.W + 4) * 8 <= 512 ? 9 : ((g.W + 4) * 8 <= 1024 ? 10 : 11);
    if ((g.W + 4) * 8 > (1 << logp)) return false;
    if (logp == 11 && (g.sh != 1 || g.dh != 1)) return false;
    bool found = false;
    for (int fn = 4; fn <= 7; ++fn) {  // 8 fragments would spill at two waves per SIMD
        if (force_fn && fn != force_fn) continue;
        // odd widths and 2048-byte lines: at most 6 fragments (the 7-fragment tile has no register to spare for them)
        if (fn == 7 && ((g.W & 1) || logp == 11)) continue;
        const int pt = (wide ? 32 : 64) * fn;
        HaloPlan p;
        p.fn = fn;
        p.logp = logp;
        p.r_max = halo_rows(pt, g.OW, OHW, g.sh, g.dh);
        const size_t per64 = (size_t)8 * p.r_max << logp;  // 64 channels = 8 octets
        if (per64 > (size_t)kMaxLdsBytes) continue;
        int cb = (int)(kMaxLdsBytes / per64) * 64;
        if (cb > cpad) cb = cpad;
        while (cpad % cb) cb -= 64;  // equal channel blocks
        p.cb = cb;
        p.lds_bytes = (size_t)(cb / 8) * p.r_max << logp;
        p.tiles_per_img = (OHW + pt - 1) / pt;
        const long wgs = (long)g.N * p.tiles_per_img * m_blocks;
        const long slots = 512;
        const long rounds = (wgs + slots - 1) / slots;
        // time ~ rounds * (work per tile + staging overhead per channel block)
        p.cost = (double)rounds * (pt + 24.0 * (cpad / cb)) / ((double)OHW * g.N * m_blocks / (double)slots);
        if (!found || p.cost < best->cost) {
            *best = p;
            found = true;
        }
    }
    return found;
}

}  // namespace

bool conv3x3_halo_supported(const ConvGeom& g, const Epilogue& ep) {
    if (!(g.kh == 3 && g.kw == 3 && g.groups == 1 && g.sh == g.sw && g.dh == g.dw)) return false;
    // stride 1 dilation 1 (any row block), or stride 2 / dilation 2 (not both) for 33 output channels and more
    const bool plain = g.sh == 1 && g.dh == 1;
    const bool variant = (g.sh == 2 && g.dh == 1) || (g.sh == 1 && g.dh == 2);
    if (!plain && !(variant && igemm_padded_rows(g.K) >= 64)) return false;
    // the LDS lines carry two zero columns on either side: padding up to the dilation (a tap never reaches further)
    if (g.ph > g.dh || g.pw > g.dw || g.C % 8) return false;
    if ((size_t)g.N * g.C * g.H * g.W >= ((size_t)1 << 31)) return false;  // 32-bit offsets
    if (pick_epilogue(ep, g.K) == EPI_GENERIC) return false;
    HaloPlan p;
    return plan_halo(g, 0, &p);
}

// the launch plan as numbers, for tests of the tile walk: fragment count, pixels per tile, tiles per image, grid.x,
// grid.y, 1 if the per-lane LDS offsets are reused across a workgroup's tiles, LDS rows per tile, channels per stage
bool conv3x3_halo_plan(const ConvGeom& g, int force_fn, int plan[8]) {
    HaloPlan p;
    if (!plan_halo(g, force_fn, &p) && !plan_halo(g, 0, &p)) return false;
    const int mpad = igemm_padded_rows(g.K);
    const int pt = (mpad > 64 ? 32 : 64) * p.fn;
    int m_blocks, grid_x;
    halo_grid(mpad, mpad > 64 ? 8 : (mpad == 64 ? 4 : 2), g.N * p.tiles_per_img, &m_blocks, &grid_x);
    plan[0] = p.fn, plan[1] = pt, plan[2] = p.tiles_per_img, plan[3] = grid_x, plan[4] = m_blocks;
    plan[5] = halo_tile_invariant(pt, g.OW, g.OH * g.OW) ? 1 : 0, plan[6] = p.r_max, plan[7] = p.cb;
    return true;
}

hipError_t run_conv3x3_halo(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                            int force_fn, hipStream_t stream) {
    HaloPlan p;
    // a forced fragment count that does not fit LDS falls back to the automatic choice
    if (!plan_halo(g, force_fn, &p) && !plan_halo(g, 0, &p)) return hipErrorInvalidValue;
    const int mpad = igemm_padded_rows(g.K);
    // the weight rows and the per-channel constants are padded to mpad rows: a workgroup must not read past them,
    // so 32 padded rows (K <= 32) take two row fragments per wave, not four
#define OHIP_HALO(FN_)                                                                  \
    case FN_:                                                                           \
        return mpad > 64    ? launch_halo<4, FN_, 2, 2>(x, wpk, out, g, ep, p, stream)  \
               : mpad == 64 ? launch_halo<4, FN_, 1, 4>(x, wpk, out, g, ep, p, stream)  \
                            : launch_halo<2, FN_, 1, 4>(x, wpk, out, g, ep, p, stream);
    switch (p.fn) {
        OHIP_HALO(4)
        OHIP_HALO(5)
        OHIP_HALO(6)
        OHIP_HALO(7)
    }
#undef OHIP_HALO
    return hipErrorInvalidValue;
}

}  // namespace ohip
