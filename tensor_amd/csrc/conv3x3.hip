// Dense int8 3x3 stride-1 convolution on the gfx950 matrix cores with the input halo resident in LDS.
//
// A workgroup owns a run of PT consecutive output pixels of one image (row-major, so a few whole output rows)
// and a block of output channels. The input rows that run touches (+1 halo row above and below, +1 zero column
// left and right) are staged into LDS ONCE, as [channel pair-of-octets][row][column][16 bytes]; after that the
// nine filter taps are nine shifted views of the same LDS tile, so every input byte is fetched from memory once
// per workgroup instead of nine times, and the main loop has no barrier at all:
//   * the MFMA "B" operand (16 input channels of one pixel) is one ds_read_b128 per lane, conflict-free because
//     the 16 lanes of a row group read 16 consecutive pixels = 256 consecutive bytes;
//   * the MFMA "A" operand (weights) is read straight from global memory, already in MFMA lane order
//     (igemm_pack_weights), one coalesced 1 KB read per 16x64 fragment, prefetched one k-chunk ahead. Every
//     workgroup reads the same <= 147 KB of weights, so they stay in L2.
// Zero padding costs nothing: the halo columns / out-of-image rows are written as zeros while staging.
#include "common.hpp"
#include <cstdlib>

#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

template <int FM, int FN, int WM, int WN, int EPI>
__global__ void __launch_bounds__(256, 2) conv3x3_halo_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk,
                                                           void* __restrict__ out, ConvGeom g, Epilogue ep, int m_tiles16,
                                                           int c_groups, int r_max, int cb, int tiles_per_img, int prm_ofs, int total_tiles,
                                                           int stagger) {
    static_assert(WM * WN == 4 && FM % 2 == 0, "four waves, row fragments in pairs");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int PT = WN * FN * 16;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    const int mt_base = blockIdx.y * (WM * FM) + wm * FM;  // first 16-row tile of this wave
    const int OHW = g.OH * g.OW;
    const int C8 = g.C / 8;
    // The per-channel epilogue constants of this workgroup's row block go to LDS now (behind the halo tile), so
    // that the epilogue does not end on a chain of global-memory round trips.
    constexpr int ROWS = WM * FM * 16;
    float* lds_prm = reinterpret_cast<float*>(lds + prm_ofs);
    for (int i = tid; i < 3 * ROWS; i += 256) {
        const int which = i / ROWS, c = blockIdx.y * ROWS + (i - which * ROWS);
        const float* src = which == 0 ? ep.scale_in : (which == 1 ? ep.bias : ep.scale_out);
        lds_prm[i] = src ? src[c] : 1.f;
    }

    // Persistent workgroups: the grid holds at most two workgroups per CU and each walks over tiles. The
    // workgroups in the second residency slot of a CU start `stagger` sleeps late, so that for the rest of the
    // kernel one workgroup's staging / epilogue (memory latency, VALU) runs under the other's MFMA phase instead
    // of both doing the same thing at the same time.
    if (stagger > 0 && ((blockIdx.x >> 8) & 1))
        for (int i = 0; i < stagger; ++i) __builtin_amdgcn_s_sleep(32);
    for (int wg0 = blockIdx.x; wg0 < total_tiles; wg0 += gridDim.x) {
        // consecutive tiles (which share halo rows) go to the same XCD / L2
        int wg = wg0;
        {
            const int per = total_tiles / 8;
            if (per > 0 && wg < per * 8) wg = (wg % 8) * per + wg / 8;
        }
        const int n = wg / tiles_per_img;
        const int t = wg % tiles_per_img;
        const int8_t* xn = x + (size_t)n * C8 * g.H * g.W * 8;
        const int p0 = t * PT;
        const int p_last = min(p0 + PT, OHW) - 1;
        const int r_lo = p0 / g.OW;
        const int R = p_last / g.OW - r_lo + 3;
        const int cols = g.W + 2;
        const int plane = r_max * cols * 16;  // bytes between channel pairs

        int bofs[FN];
#pragma unroll
        for (int f = 0; f < FN; ++f) {
            const int pix = min(p0 + (wn * FN + f) * 16 + (lane & 15), OHW - 1);
            const int oy = pix / g.OW, ox = pix % g.OW;
            bofs[f] = (oy - r_lo) * cols + ox + 1 - g.pw + (lane >> 4) * (plane / 16);  // in 16-byte units
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
            __syncthreads();  // everyone is done reading the previous channel block
            // Stage the halo: one wave per (channel pair, row) line, lanes along the columns, so that the only
            // divisions are wave-uniform (scalar) and a wave reads 2 x 512 contiguous bytes per line. Lines are taken
            // in batches of SB with all loads of a batch issued before the first LDS write, so a batch costs one
            // memory round trip.
            {
                constexpr int SB = 12;
                const int lines = (cb / 16) * R;
                for (int xc0 = 0; xc0 < cols; xc0 += 64) {
                    const int xc = xc0 + lane;
                    const int ix = xc - 1;
                    const bool col_ok = ix >= 0 && ix < g.W;
                    for (int l0 = wave; l0 < lines; l0 += 4 * SB) {
                        v2i lo[SB], hi[SB];
#pragma unroll
                        for (int k = 0; k < SB; ++k) {
                            const int line = min(l0 + 4 * k, lines - 1);
                            const int j = line / R, r = line - j * R;
                            const int iy = r_lo - g.ph + r;
                            const int o0 = cb0 / 8 + 2 * j;
                            const bool ok = col_ok && iy >= 0 && iy < g.H;
                            const int8_t* px = xn + ((size_t)iy * g.W + ix) * 8;
                            lo[k] = (ok && o0 < C8) ? *reinterpret_cast<const v2i*>(px + (size_t)o0 * g.H * g.W * 8) : v2i{0, 0};
                            hi[k] = (ok && o0 + 1 < C8) ? *reinterpret_cast<const v2i*>(px + (size_t)(o0 + 1) * g.H * g.W * 8)
                                                        : v2i{0, 0};
                        }
#pragma unroll
                        for (int k = 0; k < SB; ++k) {
                            const int line = l0 + 4 * k;
                            const int j = line / R, r = line - j * R;
                            if (line < lines && xc < cols)
                                *reinterpret_cast<v4i*>(lds + (size_t)j * plane + ((size_t)r * cols + xc) * 16) =
                                    v4i{lo[k][0], lo[k][1], hi[k][0], hi[k][1]};
                        }
                    }
                }
            }
            __syncthreads();

            // Main loop: no barrier, no branch. The nine taps are unrolled; weight fragments travel through a ring of
            // three register stages and are requested two k-chunks (~0.4 us of MFMA work) before use. Every load is
            // unconditional (the weight rows are padded to whole row blocks and the chunk index is clamped), so that
            // the compiler can count outstanding loads and wait only for the oldest stage.
            v4i ring[3][FM];
            const int cg0 = cb0 / 64;
            auto load_a = [&](int cc, int tap, v4i (&a)[FM]) {
                const int8_t* p = wlane + (size_t)(tap * c_groups + cg0 + cc) * kc_stride;
#pragma unroll
                for (int i = 0; i < FM; ++i) a[i] = *reinterpret_cast<const v4i*>(p + i * 1024);
            };
            load_a(0, 0, ring[0]);
            load_a(0, 1, ring[1]);
            for (int cc = 0; cc < nck; ++cc) {
                const int cc_next = min(cc + 1, nck - 1);
                const int ccofs = cc * 4 * (plane / 16);
#pragma unroll
                for (int tap = 0; tap < 9; ++tap) {
                    if (tap + 2 < 9) load_a(cc, tap + 2, ring[(tap + 2) % 3]);
                    else load_a(cc_next, tap + 2 - 9, ring[(tap + 2) % 3]);
                    const int tapofs = (tap / 3) * cols + tap % 3 + ccofs;  // 16-byte units: keeps ds_read_b128
                    v4i b[FN];
#pragma unroll
                    for (int f = 0; f < FN; ++f) b[f] = reinterpret_cast<const v4i*>(lds)[bofs[f] + tapofs];
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int f = 0; f < FN; ++f)
                            acc[i][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[tap % 3][i], b[f], acc[i][f], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);  // keep the prefetch distance: no hoisting of later taps' loads
                }
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
                const int cl = ch0 - blockIdx.y * ROWS;  // channel within the row block
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    prm.si[e] = lds_prm[cl + e];
                    prm.bi[e] = lds_prm[ROWS + cl + e];
                    prm.so[e] = lds_prm[2 * ROWS + cl + e];
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
    int fn, r_max, cb, tiles_per_img;
    size_t lds_bytes;
    double cost;
};

// rows of output a run of pt pixels starting at a multiple of pt can touch, +2 halo rows
int halo_rows(int pt, int OW, int OHW) {
    int worst = 0;
    for (int p0 = 0; p0 < OHW; p0 += pt) {
        const int last = (p0 + pt < OHW ? p0 + pt : OHW) - 1;
        const int rows = last / OW - p0 / OW + 3;
        if (rows > worst) worst = rows;
    }
    return worst;
}

template <int FM, int FN, int WM, int WN, int EPI>
hipError_t launch_halo_e(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const HaloPlan& pl, hipStream_t stream) {
    auto kern = conv3x3_halo_kernel<FM, FN, WM, WN, EPI>;
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kMaxLdsBytes + kPrmLdsBytes);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int mpad = igemm_padded_rows(g.K);
    const int m_blocks = (mpad / 16 + WM * FM - 1) / (WM * FM);
    const int prm_ofs = (int)((pl.lds_bytes + 15) / 16 * 16);
    const int total_tiles = g.N * pl.tiles_per_img;
    int grid_x = 512 / m_blocks;  // two resident workgroups per CU
    if (grid_x < 8) grid_x = 8;
    if (grid_x > total_tiles) grid_x = total_tiles;
    // stagger only pays when every slot has at least two tiles to walk through
    static const char* env = getenv("OHIP_HALO_STAGGER");
    const int stagger = env ? atoi(env) : 0;
    hipLaunchKernelGGL(kern, dim3(grid_x, m_blocks), dim3(256), prm_ofs + 3 * WM * FM * 16 * sizeof(float), stream, x, wpk,
                       out, g, ep, mpad / 16, igemm_channel_groups(g.C), pl.r_max, pl.cb, pl.tiles_per_img, prm_ofs,
                       total_tiles, (grid_x == 512 / m_blocks && grid_x >= 512) ? stagger : 0);
    return hipGetLastError();
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
        return launch_halo_e<FM, FN, WM, WN, EPI_GENERIC>(x, wpk, out, g, ep, pl, stream);
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
    bool found = false;
    for (int fn = 4; fn <= 7; ++fn) {  // 8 fragments would spill at two waves per SIMD
        if (force_fn && fn != force_fn) continue;
        const int pt = (wide ? 32 : 64) * fn;
        HaloPlan p;
        p.fn = fn;
        p.r_max = halo_rows(pt, g.OW, OHW);
        const size_t per64 = (size_t)64 * p.r_max * (g.W + 2);
        if (per64 > (size_t)kMaxLdsBytes) continue;
        int cb = (int)(kMaxLdsBytes / per64) * 64;
        if (cb > cpad) cb = cpad;
        while (cpad % cb) cb -= 64;  // equal channel blocks
        p.cb = cb;
        p.lds_bytes = (size_t)cb * p.r_max * (g.W + 2);
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

bool conv3x3_halo_supported(const ConvGeom& g) {
    if (!(g.kh == 3 && g.kw == 3 && g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.groups == 1)) return false;
    if (g.ph > 1 || g.pw > 1 || g.C % 8) return false;
    HaloPlan p;
    return plan_halo(g, 0, &p);
}

hipError_t run_conv3x3_halo(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                            int force_fn, hipStream_t stream) {
    HaloPlan p;
    if (!plan_halo(g, force_fn, &p)) return hipErrorInvalidValue;
    const bool wide = igemm_padded_rows(g.K) > 64;
#define OHIP_HALO(FN_)                                                                  \
    case FN_:                                                                           \
        return wide ? launch_halo<4, FN_, 2, 2>(x, wpk, out, g, ep, p, stream)          \
                    : launch_halo<4, FN_, 1, 4>(x, wpk, out, g, ep, p, stream);
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
