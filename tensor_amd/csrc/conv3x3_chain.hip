// A chain of dense int8 3x3 stride-1 "same" convolutions (each int8 Byte8 -> int8 Byte8, same shape, 33..128 channels)
// as ONE persistent launch of the LDS-halo kernel of conv3x3.hip.
//
// Launched one by one, every layer pays its own ramp and drain, and a layer whose tile count is not a multiple of the
// resident workgroups leaves compute units idle at its end (64 images of 56x56: 896 tiles on 512 workgroups = 1.75
// rounds; four layers = 3584 tiles = exactly 7 each). Here the workgroups walk ONE list of tiles that runs through
// all layers; a tile of layer l starts as soon as the (at most three) tiles of layer l-1 that wrote its input rows are
// done, so the layers overlap at their seams.
//
//   * Dependencies are kept inside an XCD. Each XCD has its own L2; what one compute unit wrote is visible to the
//     others of the SAME XCD as soon as the store has been acknowledged (s_waitcnt vmcnt(0)), with no cache
//     maintenance. So the images are dealt to the XCDs (image n belongs to XCD n % xcds), every XCD has its own tile
//     list (layer-major: all its tiles of layer 0, then layer 1, ...) and its own queue counter, and a workgroup
//     reads the XCD it really runs on from the hardware register, whatever the dispatch order was.
//   * A workgroup takes the next tile of its XCD's list with an atomic counter. Before it stages a tile's input
//     rows it needs the producer tiles' flags (flag == the launch's epoch number). The check for the NEXT tile is made
//     without waiting while the current tile is still in flight (then the transfer runs under the epilogue, as in
//     the per-layer kernel); if the producers are not done yet, the workgroup first finishes and publishes its
//     current tile and only then waits. A waiting workgroup therefore never holds an unpublished tile, and since
//     tiles are taken in list order by workgroups that are all resident, the oldest unfinished tile can always run:
//     no cycle of waits. Every wait is bounded: after 2^17 polls the workgroup gives up, raises the error word and
//     goes on (wrong results, reported by the host), so the grid always drains.
//   * A tile's flag is set by one thread after the barrier at the top of the workgroup's next tile: every wave has
//     passed s_waitcnt vmcnt(0) by then, so all of the tile's stores have been acknowledged by L2.
//   * Each layer writes a buffer nobody has read before in this launch (the caller provides layers - 1 intermediate
//     buffers), so a compute unit's vector L1 cannot hold a stale line of what it is about to read.
#include <atomic>
#include <mutex>

#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

namespace {

constexpr unsigned CHAIN_OOB = 0x80000000u;  // beyond the buffer descriptor: reads as zero
// cache policy of the halo transfers: sc1 (agent scope) = the load does not hit in the compute unit's own vector L1, which
// could hold a line fetched while a neighbouring producer tile had not written its share of it yet
constexpr int CHAIN_LOAD_AUX = 1 << 4;
constexpr int CHAIN_MAX_LAYERS = 8;
constexpr int CHAIN_MAX_FLAGS = 1 << 16;   // tiles of all layers
constexpr int CHAIN_SPIN_LIMIT = 1 << 17;  // polls of a producer flag before giving up (~0.1 s)

// per-device state of the chain launches: tile flags (epoch numbers), one queue counter per XCD, exit counter, error word
// One set of flags and counters per stream that uses the entry point, for up to CHAIN_SLOTS streams per GPU: launches on
// different streams may overlap and must not share them.
constexpr int CHAIN_SLOTS = 4;
__device__ int g_chain_flags[CHAIN_SLOTS * CHAIN_MAX_FLAGS];
__device__ int g_chain_ctl[CHAIN_SLOTS * 16];  // per slot: [0..7] queue counters, [8] workgroups that have left, [9] error, [10] launches completed,
                                               // [11] shader cycles and [12] ticks of the 100 MHz counter of the last launch (its last workgroup's life)

struct ChainArgs {
    const int8_t* act[CHAIN_MAX_LAYERS + 1];  // act[l]: input of layer l; act[l + 1]: its output
    const int8_t* wpk[CHAIN_MAX_LAYERS];
    const float* scale_in[CHAIN_MAX_LAYERS];
    const float* bias[CHAIN_MAX_LAYERS];
    const float* scale_out[CHAIN_MAX_LAYERS];
    float act_hi[CHAIN_MAX_LAYERS], act_p0[CHAIN_MAX_LAYERS];
    int lrelu[CHAIN_MAX_LAYERS];
    int layers, xcds;
    int* flags;
    int* ctl;
};

__device__ __forceinline__ int chain_xcc_id() {
    // HW_REG_XCC_ID (id 20), bits 3:0: the accelerator complex die this wave runs on
    return (int)__builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11));
}

}  // namespace

// FM = 4 row fragments per wave; waves = WM (channel blocks of 64) x 4 / WM (pixel blocks): WM = 2 for 65..128 output
// channels (128 channels x 32*FN pixels per tile), WM = 1 for 33..64 (64 channels x 64*FN pixels), the whole reduction
// staged at once (C = K <= 128 here). See conv3x3.hip for the data path.
template <int FN, int EPI, int LOGP, int WM>
__global__ void __launch_bounds__(256, 2) conv3x3_chain_kernel(ConvGeom g, Epilogue ep0, ChainArgs ca, int m_tiles16,
                                                            int c_groups, int r_max, int tiles_per_img,
                                                            unsigned act_bytes) {
    constexpr int FM = 4, WN = 4 / WM;
    constexpr bool NONNEG = EPI == EPI_I8_P8_NONNEG;
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int PT = WN * FN * 16;
    constexpr int PITCH = 1 << LOGP;
    constexpr int ROWS = WM * FM * 16;  // 128 or 64
    __shared__ __attribute__((aligned(16))) float lds_prm[3 * ROWS];
    __shared__ int lds_ctl[4];  // [0] next tile index (-1: none), [1] its producers are done

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int mt_base = wm * FM;
    const int OHW = g.OH * g.OW;
    const int C8 = g.C / 8;
    const int EW = g.W + 4;
    const int pair_bytes = r_max * 2 * PITCH;
    const int cb = c_groups * 64;
    const unsigned inv_ow20 = ((1u << 20) + (unsigned)g.OW - 1u) / (unsigned)g.OW;  // ceil(2^20 / OW), uniform

    // The launch's epoch number = the count of completed launches on this flag set + 1, kept in device memory (ctl[10],
    // advanced by the last workgroup to leave): a launch replayed from a captured graph gets a fresh number like any other.
    const int epoch = __builtin_amdgcn_readfirstlane(__hip_atomic_load(ca.ctl + 10, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) + 1;
    // (for the clock the kernel ran at: the shader-cycle counter and the constant 100 MHz counter, read again by the last
    // workgroup to leave)
    const unsigned long long clk0 = __builtin_readcyclecounter(), ref0 = __builtin_amdgcn_s_memrealtime();

    // ---- this XCD's tile list ------------------------------------------------------------------------------------
    const int xcd = __builtin_amdgcn_readfirstlane(chain_xcc_id() % ca.xcds);
    const int my_images = (g.N - xcd + ca.xcds - 1) / ca.xcds;  // images xcd, xcd + xcds, ...
    const int per_layer = my_images * tiles_per_img;
    const int list_len = per_layer * ca.layers;
    struct Tile {
        int l, n, t;
    };
    auto tile_at = [&](int i) {
        Tile tl;
        tl.l = i / per_layer;
        const int r = i - tl.l * per_layer;
        const int m = r / tiles_per_img;
        tl.t = r - m * tiles_per_img;
        tl.n = xcd + m * ca.xcds;
        return tl;
    };
    auto flag_of = [&](int l, int n, int t) { return ca.flags + ((size_t)l * g.N + n) * tiles_per_img + t; };
    // producers of tile (l, n, t): the tiles of layer l-1 that hold input rows r_lo-1 .. r_hi+1 of image n
    auto producers = [&](const Tile& tl, int& t_lo, int& t_hi) {
        const int p0 = tl.t * PT, p_last = min(p0 + PT, OHW) - 1;
        const int row_lo = max(p0 / g.OW - 1, 0), row_hi = min(p_last / g.OW + 1, g.OH - 1);
        t_lo = row_lo * g.OW / PT;
        t_hi = (row_hi * g.OW + g.OW - 1) / PT;
    };
    auto deps_ready = [&](const Tile& tl) -> bool {  // one poll of every producer flag
        if (tl.l == 0) return true;
        int t_lo, t_hi;
        producers(tl, t_lo, t_hi);
        // at most three producers (a tile's rows +-1 reach into the tile before and the tile behind): their flags are
        // requested together, one round trip to L2 instead of up to three in a row
        const int* f = flag_of(tl.l - 1, tl.n, 0);
        const int t_mid = min(t_lo + 1, t_hi);
        const int v0 = __hip_atomic_load(f + t_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int v1 = __hip_atomic_load(f + t_mid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int v2 = __hip_atomic_load(f + t_hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bool ok = v0 == epoch && v1 == epoch && v2 == epoch;
        for (int t = t_lo + 2; t < t_hi; ++t)  // (only tiles shorter than an image row have more producers)
            ok = ok && __hip_atomic_load(f + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == epoch;
        return ok;
    };
    auto deps_wait = [&](const Tile& tl) {  // thread 0 only; bounded
        for (int spin = 0; spin < CHAIN_SPIN_LIMIT; ++spin) {
            if (deps_ready(tl)) return;
            __builtin_amdgcn_s_sleep(8);
        }
        __hip_atomic_store(ca.ctl + 9, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // gave up: results are wrong
    };
    auto grab = [&]() -> int {  // thread 0 only
        const int i = __hip_atomic_fetch_add(ca.ctl + xcd, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return i < list_len ? i : -1;
    };

    // ---- halo transfer of one tile (as in conv3x3.hip; the whole reduction in one stage) ---------------------------
    auto stage = [&](const Tile& tl) {
        const __amdgpu_buffer_rsrc_t rin =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(ca.act[tl.l]), 0, (int)act_bytes, 0x00020000);
        const int n = tl.n, p0 = tl.t * PT;
        const int p_last = min(p0 + PT, OHW) - 1;
        const int r_lo = p0 / g.OW;
        const int R = p_last / g.OW - r_lo + 3;
        if constexpr (LOGP == 9) {
            const int hl = lane >> 5, pp = lane & 31;
            const bool col_ok = pp >= 1 && 2 * pp - 2 < g.W;
            const unsigned v_px = (unsigned)(2 * pp - 2) * 8u;
            const unsigned v_both = col_ok ? v_px + (unsigned)hl * (unsigned)(g.H * g.W * 8) : CHAIN_OOB;
            const unsigned v_first = (col_ok && hl == 0) ? v_px : CHAIN_OOB;
            if (2 * pp < EW) {
                for (int pj = wave; pj < cb / 16; pj += 4) {
                    const int o = 2 * pj;
                    const bool both = o + 1 < C8;
                    for (int r = 0; r < R; ++r) {
                        const int iy = r_lo - g.ph + r;
                        const bool ok = o < C8 && iy >= 0 && iy < g.H;
                        const unsigned s_off = ok ? (unsigned)((n * C8 + o) * g.H + iy) * (unsigned)(g.W * 8) : 0u;
                        int8_t* dst = lds + (size_t)pj * pair_bytes + (size_t)((2 * r) << LOGP);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, (__attribute__((address_space(3))) void*)dst, 16,
                                                                 (int)(ok ? (both ? v_both : v_first) : CHAIN_OOB), (int)s_off,
                                                                 0, CHAIN_LOAD_AUX);
                    }
                }
            }
        } else {
            const bool col_ok = lane >= 1 && 2 * lane - 2 < g.W;
            const unsigned v_col = col_ok ? (unsigned)(2 * lane - 2) * 8u : CHAIN_OOB;
            if (2 * lane < EW) {
                for (int oc = wave; oc < cb / 8; oc += 4) {
                    for (int r = 0; r < R; ++r) {
                        const int iy = r_lo - g.ph + r;
                        const bool ok = oc < C8 && iy >= 0 && iy < g.H;
                        const unsigned s_off = ok ? (unsigned)((n * C8 + oc) * g.H + iy) * (unsigned)(g.W * 8) : 0u;
                        int8_t* dst = lds + (size_t)(oc >> 1) * pair_bytes + (size_t)((2 * r + (oc & 1)) << LOGP);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rin, (__attribute__((address_space(3))) void*)dst, 16,
                                                                 (int)(ok ? v_col : CHAIN_OOB), (int)s_off, 0, CHAIN_LOAD_AUX);
                    }
                }
            }
        }
    };
    // odd width: see conv3x3.hip
    auto fix_odd = [&](int p0) {
        if (!(g.W & 1)) return;
        const int p_last = min(p0 + PT, OHW) - 1;
        const int R = p_last / g.OW - p0 / g.OW + 3;
        const int lines = (cb / 8) * R;
        for (int i = lane; i < lines; i += 64) {
            const int oc = i / R, r = i - oc * R;
            const int owner = LOGP == 9 ? (oc >> 1) & 3 : oc & 3;
            if (owner != wave) continue;
            int8_t* line = lds + (size_t)(oc >> 1) * pair_bytes + (size_t)((2 * r + (oc & 1)) << LOGP);
            *reinterpret_cast<v2i*>(line + (g.W + 2) * 8) = v2i{0, 0};
        }
    };

    // ---- first tile ------------------------------------------------------------------------------------------------
    if (tid == 0) {
        const int i = grab();
        if (i >= 0) deps_wait(tile_at(i));  // (no unpublished tile held: waiting is safe)
        lds_ctl[0] = i;
    }
    __syncthreads();
    int cur_i = lds_ctl[0];
    if (cur_i >= 0) stage(tile_at(cur_i));
    int prm_layer = -1;
    int done_i = -1;  // tile whose stores are out but whose flag is not set yet

    while (cur_i >= 0) {
        const Tile tl = tile_at(cur_i);
        const int n = tl.n, p0 = tl.t * PT;
        const int r_lo = p0 / g.OW;
        Epilogue ep = ep0;
        ep.scale_in = ca.scale_in[tl.l], ep.bias = ca.bias[tl.l], ep.scale_out = ca.scale_out[tl.l];
        ep.act_hi = ca.act_hi[tl.l], ep.act_p0 = ca.act_p0[tl.l], ep.lrelu = ca.lrelu[tl.l] != 0;

        // LDS offset of each fragment's pixel (tap 0, 0). Row and column relative to the tile's first row come from a
        // multiplication by 2^20 / OW (exact: (column of the first pixel + offset in the tile) * OW < 2^20, both factors
        // below 2^24), not from a division per fragment: seven 32-bit divisions were a tenth of a tile's vector work.
        int bcc[FN];
        const int col0 = p0 - r_lo * g.OW;                 // column of the tile's first pixel (uniform)
        const int rel_max = min(p0 + PT, OHW) - 1 - p0 + col0;  // lanes past the image end keep the last pixel
#pragma unroll
        for (int f = 0; f < FN; ++f) {
            const int rel = min(col0 + (wn * FN + f) * 16 + (lane & 15), rel_max);
            const int oy_rel = (int)(__umul24((unsigned)rel, inv_ow20) >> 20);
            const int ox = rel - oy_rel * g.OW;
            bcc[f] = oy_rel * 2 * PITCH + (ox - g.pw + 2) * 8 + (lane >> 4) * pair_bytes;
        }
        v4i acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int f = 0; f < FN; ++f) acc[i][f] = v4i{0, 0, 0, 0};

        const int nck = cb / 64;
        const int8_t* wlane = ca.wpk[tl.l] + ((size_t)mt_base * 64 + lane) * 16;
        const size_t kc_stride = (size_t)m_tiles16 * 1024;
        constexpr int RD = FN >= 7 ? 2 : 3;
        v4i ring[RD][FM];
        auto a_ptr = [&](int cc, int tap) { return wlane + (size_t)(tap * c_groups + cc) * kc_stride; };
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
        // this tile's rows were requested a tile ago: wait for this wave's transfers (and, with them, for every store of
        // the previous tile's epilogue), then for everyone's
        __builtin_amdgcn_s_waitcnt(0);
        fix_odd(p0);
        __syncthreads();
        // every wave's stores of the previous tile have been acknowledged: publish it
        if (tid == 0 && done_i >= 0) {
            const Tile d = tile_at(done_i);
            __hip_atomic_store(flag_of(d.l, d.n, d.t), epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        done_i = -1;
        // the epilogue constants of this tile's layer (nobody reads the old ones any more; the barrier behind the
        // matrix loop orders these writes before the epilogue's reads)
        if (prm_layer != tl.l) {
            for (int i = tid; i < 3 * ROWS; i += 256) {
                const int which = i / ROWS, c = i - which * ROWS;
                const float* src = which == 0 ? ep.scale_in : (which == 1 ? ep.bias : ep.scale_out);
                lds_prm[i] = src[c];
            }
            prm_layer = tl.l;
        }

        // the next tile of this XCD's list: requested now, needed behind the matrix loop (thread 0; the others carry -1)
        int nxt_pre = -1;
        if (tid == 0) nxt_pre = grab();

        load_a(0, 0, ring[0]);
        if constexpr (RD == 3) load_a(0, 1, ring[1]);
        v4i b[FN];
#pragma unroll
        for (int f = 0; f < FN; ++f) b[f] = read_b(bcc[f]);
        for (int cc = 0; cc < nck; ++cc) {
            const int cc_next = min(cc + 1, nck - 1);
            const int to_next = (cc_next - cc) * 4 * pair_bytes;
#pragma unroll
            for (int tap = 0; tap < 9; ++tap) {
                constexpr int AH = RD - 1;
                const int8_t* pa = tap + AH < 9 ? a_ptr(cc, tap + AH) : a_ptr(cc_next, tap + AH - 9);
                constexpr int kRowB = 2 * PITCH;
                const int nofs = tap < 8 ? ((tap + 1) / 3) * kRowB + ((tap + 1) % 3) * 8 : 0;
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
#pragma unroll
                for (int i = 0; i < FM; ++i) ring[0][i] = ring[1][i];
            }
        }
        // whether the next tile's producers are done by now (one poll, no waiting: this workgroup still holds an
        // unpublished tile)
        if (tid == 0) {
            lds_ctl[0] = nxt_pre;
            lds_ctl[1] = (nxt_pre >= 0 && deps_ready(tile_at(nxt_pre))) ? 1 : 0;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no weight fragment pending when the transfers are issued
        __syncthreads();                     // everyone is done reading LDS; lds_ctl is visible
        const int nxt_i = lds_ctl[0];
        const bool early = lds_ctl[1] != 0;
        if (nxt_i >= 0 && early) stage(tile_at(nxt_i));  // runs under the epilogue

        // ---- epilogue ------------------------------------------------------------------------------------------------
        const int gq = lane >> 4;
        int8_t* out = const_cast<int8_t*>(ca.act[tl.l + 1]);
#pragma unroll
        for (int ip = 0; ip < FM / 2; ++ip) {
            const int ch0 = 32 * (mt_base / 2 + ip) + 8 * gq;
            const bool ch_ok = ch0 < g.K;
            Epi8 prm;
            const unsigned pa = (unsigned)(size_t)(__attribute__((address_space(3))) float*)lds_prm + (unsigned)ch0 * 4u;
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
            if constexpr (NONNEG) epi8_clamp_init(ep, prm);
#pragma unroll
            for (int f = 0; f < FN; ++f) {
                const int pix = p0 + (wn * FN + f) * 16 + (lane & 15);
                int a8[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a8[e] = acc[2 * ip][f][e];
                    a8[4 + e] = acc[2 * ip + 1][f][e];
                }
                if (ch_ok && pix < OHW) epi8_store_i8p8<NONNEG>(out, ep, prm, elem_offset(8, n, ch0, pix, g.K, OHW), a8);
            }
        }
        done_i = cur_i;

        if (nxt_i >= 0 && !early) {
            // the producers were not done: publish this tile first (so that nobody can be waiting for a tile held by a
            // waiting workgroup), then wait, then request the rows
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            if (tid == 0) {
                __hip_atomic_store(flag_of(tl.l, tl.n, tl.t), epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                deps_wait(tile_at(nxt_i));
            }
            done_i = -1;
            __syncthreads();
            stage(tile_at(nxt_i));
        }
        cur_i = nxt_i;
    }
    // the last tile of this workgroup
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        if (done_i >= 0) {
            const Tile d = tile_at(done_i);
            __hip_atomic_store(flag_of(d.l, d.n, d.t), epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // the last workgroup to leave rewinds the queues for the next launch
        const int left = __hip_atomic_fetch_add(ca.ctl + 8, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            // every list must have been walked to its end: a list whose XCD received no workgroup of this launch would
            // otherwise go unnoticed (the host sizes the grid so that this does not happen; the status call reports it)
            for (int xc = 0; xc < ca.xcds; ++xc) {
                const int len = ((g.N - xc + ca.xcds - 1) / ca.xcds) * tiles_per_img * ca.layers;
                if (__hip_atomic_load(ca.ctl + xc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < len)
                    __hip_atomic_store(ca.ctl + 9, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            for (int i = 0; i < 9; ++i) __hip_atomic_store(ca.ctl + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ca.ctl[11] = (int)(__builtin_readcyclecounter() - clk0);
            ca.ctl[12] = (int)(__builtin_amdgcn_s_memrealtime() - ref0);
            __hip_atomic_store(ca.ctl + 10, epoch == 0x7ffffffe ? 0 : epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------

namespace {

constexpr int kChainLdsBytes = 64 * 1024;
constexpr int kChainPrmBytes = 3 * 128 * 4 + 64;

struct ChainDevice {
    int* flags = nullptr;
    int* ctl = nullptr;
    int xcds = 0;
    // A flag set (slot) belongs to the stream that launched on it last. A stream that has none takes a free slot, or the
    // least recently used one whose last launch has completed (its event says so): a caller that rotates through more
    // streams than there are slots keeps the single launch as long as at most CHAIN_SLOTS of them are busy at a time.
    // A slot handed to a stream under graph capture is baked into the graph and stays with that stream for good.
    hipStream_t stream[CHAIN_SLOTS] = {};
    bool used[CHAIN_SLOTS] = {};
    bool pinned[CHAIN_SLOTS] = {};
    hipEvent_t done[CHAIN_SLOTS] = {};
    unsigned long stamp[CHAIN_SLOTS] = {};
    unsigned long clock = 0;
};
ChainDevice g_chain_dev[16];
std::mutex g_chain_mutex;  // slot table, launches and the status read-and-rewind

}  // namespace

// can this chain of layers (same geometry g for all) run as one launch? `plan` receives {fragments, lds rows, tiles per image, line pitch log2}
bool conv3x3_chain_applicable(const ConvGeom& g, const Epilogue& ep, int layers, int plan[4], int force_fn) {
    if (layers < 2 || layers > CHAIN_MAX_LAYERS) return false;
    if (g.C != g.K || g.ph != 1 || g.pw != 1 || g.OH != g.H || g.OW != g.W) return false;
    if (g.sh != 1 || g.sw != 1 || g.dh != 1 || g.dw != 1) return false;
    if ((g.W + 4) * 8 > 1024) return false;  // LDS lines of 512 and 1024 bytes only
    if (igemm_padded_rows(g.K) != 128 && igemm_padded_rows(g.K) != 64) return false;  // 33..128 channels: one row block
    if (!conv3x3_halo_supported(g, ep)) return false;
    const int epi = pick_epilogue(ep, g.K);
    if (epi != EPI_I8_P8 && epi != EPI_I8_P8_NONNEG) return false;
    int hp[8];
    if (!conv3x3_halo_plan(g, force_fn, hp)) return false;  // (a forced fragment count that does not fit: the automatic one)
    if (hp[7] != igemm_channel_groups(g.C) * 64) return false;  // the whole reduction must fit one LDS stage
    if ((long)layers * g.N * hp[2] > CHAIN_MAX_FLAGS) return false;
    plan[0] = hp[0], plan[1] = hp[6], plan[2] = hp[2], plan[3] = (g.W + 4) * 8 <= 512 ? 9 : 10;
    return true;
}

hipError_t run_conv3x3_chain(const ConvGeom& g, const Epilogue* eps, const int8_t* const* wpk, const int8_t* const* act,
                             int layers, int* error_word_out, hipStream_t stream, int force_fn) {
    int plan[4];
    if (!conv3x3_chain_applicable(g, eps[0], layers, plan, force_fn)) return hipErrorInvalidValue;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
    ChainDevice& cd = g_chain_dev[dev];
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if ((e = hipStreamIsCapturing(stream, &cs)) != hipSuccess) return e;
    const bool capturing = cs != hipStreamCaptureStatusNone;
    // the launch itself is made under the lock as well: conv3x3_chain_error rewinds the queues of every slot from the
    // host and must not meet a launch that another thread enqueues in between
    std::lock_guard<std::mutex> lock(g_chain_mutex);
    int slot = -1;
    {
        if (!cd.flags) {
            void *pf = nullptr, *pc = nullptr;
            if ((e = hipGetSymbolAddress(&pf, HIP_SYMBOL(g_chain_flags))) != hipSuccess) return e;
            if ((e = hipGetSymbolAddress(&pc, HIP_SYMBOL(g_chain_ctl))) != hipSuccess) return e;
            hipDeviceProp_t prop;
            if ((e = hipGetDeviceProperties(&prop, dev)) != hipSuccess) return e;
            cd.flags = (int*)pf, cd.ctl = (int*)pc;
            cd.xcds = std::max(1, std::min(8, prop.multiProcessorCount / 32));
        }
        for (int i = 0; i < CHAIN_SLOTS && slot < 0; ++i)
            if (cd.used[i] && cd.stream[i] == stream) slot = i;
        for (int i = 0; i < CHAIN_SLOTS && slot < 0; ++i)
            if (!cd.used[i]) slot = i;
        if (slot < 0) {
            // every slot has an owner: the one that has been idle longest, if its last launch has completed
            int lru = -1;
            for (int i = 0; i < CHAIN_SLOTS; ++i)
                if (!cd.pinned[i] && (lru < 0 || cd.stamp[i] < cd.stamp[lru])) lru = i;
            for (int k = 0; k < CHAIN_SLOTS && slot < 0 && lru >= 0; ++k) {
                const int i = (lru + k) % CHAIN_SLOTS;
                if (cd.pinned[i] || !cd.done[i]) continue;
                const hipError_t q = hipEventQuery(cd.done[i]);
                if (q == hipSuccess) slot = i;
                else if (q != hipErrorNotReady) return q;
            }
            if (slot < 0) return hipErrorNotReady;  // all busy: the caller runs the layers one by one
        }
        if (!cd.done[slot] && (e = hipEventCreateWithFlags(&cd.done[slot], hipEventDisableTiming)) != hipSuccess) return e;
        cd.used[slot] = true, cd.stream[slot] = stream;
        cd.pinned[slot] = cd.pinned[slot] || capturing;
        cd.stamp[slot] = ++cd.clock;
    }
    ChainArgs ca;
    for (int l = 0; l < layers; ++l) {
        ca.act[l] = act[l];
        ca.wpk[l] = wpk[l];
        ca.scale_in[l] = eps[l].scale_in, ca.bias[l] = eps[l].bias, ca.scale_out[l] = eps[l].scale_out;
        ca.act_hi[l] = eps[l].act_hi, ca.act_p0[l] = eps[l].act_p0, ca.lrelu[l] = eps[l].lrelu ? 1 : 0;
    }
    ca.act[layers] = act[layers];
    ca.layers = layers, ca.xcds = cd.xcds;
    ca.flags = cd.flags + (size_t)slot * CHAIN_MAX_FLAGS, ca.ctl = cd.ctl + slot * 16;
    const int fn = plan[0], r_max = plan[1], tpi = plan[2], logp = plan[3];
    const int epi = pick_epilogue(eps[0], g.K);
    const unsigned act_bytes = (unsigned)((size_t)g.N * g.C * g.H * g.W);
    const size_t lds_bytes = (size_t)(igemm_channel_groups(g.C) * 8) * r_max << logp;
    const long total = (long)layers * g.N * tpi;
    const int grid = (int)std::min<long>(512, std::max<long>(total, 8));
#define OHIP_CHAIN_W(FN_, E_, P_, W_)                                                                                  \
    do {                                                                                                               \
        auto kern = conv3x3_chain_kernel<FN_, E_, P_, W_>;                                                             \
        static std::atomic<bool> attr_set[16] = {};                                                                    \
        if (!attr_set[dev].load(std::memory_order_acquire)) {                                                          \
            hipError_t e2 = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,        \
                                                kChainLdsBytes + kChainPrmBytes);                                      \
            if (e2 != hipSuccess) return e2;                                                                           \
            attr_set[dev].store(true, std::memory_order_release);                                                      \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, g, eps[0], ca, igemm_padded_rows(g.K) / 16, \
                           igemm_channel_groups(g.C), r_max, tpi, act_bytes);                                          \
    } while (0)
#define OHIP_CHAIN(FN_, E_, P_)                                  \
    do {                                                         \
        if (igemm_padded_rows(g.K) == 128) OHIP_CHAIN_W(FN_, E_, P_, 2); \
        else OHIP_CHAIN_W(FN_, E_, P_, 1);                       \
    } while (0)
#define OHIP_CHAIN_P(FN_, E_)                   \
    do {                                        \
        if (logp == 9) OHIP_CHAIN(FN_, E_, 9);  \
        else OHIP_CHAIN(FN_, E_, 10);           \
    } while (0)
#define OHIP_CHAIN_E(FN_)                                                 \
    do {                                                                  \
        if (epi == EPI_I8_P8_NONNEG) OHIP_CHAIN_P(FN_, EPI_I8_P8_NONNEG); \
        else OHIP_CHAIN_P(FN_, EPI_I8_P8);                                \
    } while (0)
    switch (fn) {
    case 4: OHIP_CHAIN_E(4); break;
    case 5: OHIP_CHAIN_E(5); break;
    case 6: OHIP_CHAIN_E(6); break;
    default: OHIP_CHAIN_E(7); break;
    }
#undef OHIP_CHAIN_E
#undef OHIP_CHAIN_P
#undef OHIP_CHAIN
#undef OHIP_CHAIN_W
    if (error_word_out) *error_word_out = 0;
    if ((e = hipGetLastError()) != hipSuccess) return e;
    // (no event inside a capture: the slot is pinned to the stream then and never asked for its state)
    return capturing ? hipSuccess : hipEventRecord(cd.done[slot], stream);
}

// the error word of the last chain launches on this device (1: a workgroup gave up waiting for a producer tile);
// synchronizes with the device and clears it. Launches on other host threads wait at the lock meanwhile, so the rewind
// cannot meet a launch in flight.
hipError_t conv3x3_chain_error(int* error_word) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    *error_word = 0;
    std::lock_guard<std::mutex> lock(g_chain_mutex);
    if ((e = hipDeviceSynchronize()) != hipSuccess) return e;
    if (dev < 0 || dev >= 16 || !g_chain_dev[dev].ctl) return hipSuccess;
    int ctl[CHAIN_SLOTS * 16];
    if ((e = hipMemcpy(ctl, g_chain_dev[dev].ctl, sizeof(ctl), hipMemcpyDeviceToHost)) != hipSuccess) return e;
    bool dirty = false;
    for (int s = 0; s < CHAIN_SLOTS; ++s) {
        *error_word |= ctl[s * 16 + 9];
        dirty = dirty || ctl[s * 16 + 9] || ctl[s * 16 + 8] || ctl[s * 16];
    }
    if (dirty) {  // a launch that gave up (or was cut short) leaves the counters dirty: rewind them, keep the launch counts
        for (int s = 0; s < CHAIN_SLOTS; ++s)
            for (int i = 0; i < 10; ++i) ctl[s * 16 + i] = 0;
        if ((e = hipMemcpy(g_chain_dev[dev].ctl, ctl, sizeof(ctl), hipMemcpyHostToDevice)) != hipSuccess) return e;
    }
    return hipSuccess;
}

// the shader clock of the most recent single-launch chain on this device, from the two counters its last workgroup
// left behind; synchronizes with the device. 0 if there has been none.
hipError_t conv3x3_chain_clock_mhz(float* mhz) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    *mhz = 0.f;
    std::lock_guard<std::mutex> lock(g_chain_mutex);
    if ((e = hipDeviceSynchronize()) != hipSuccess) return e;
    if (dev < 0 || dev >= 16 || !g_chain_dev[dev].ctl) return hipSuccess;
    int ctl[CHAIN_SLOTS * 16];
    if ((e = hipMemcpy(ctl, g_chain_dev[dev].ctl, sizeof(ctl), hipMemcpyDeviceToHost)) != hipSuccess) return e;
    int best = -1;
    for (int s = 0; s < CHAIN_SLOTS; ++s)
        if (g_chain_dev[dev].used[s] && ctl[s * 16 + 12] > 0 && (best < 0 || g_chain_dev[dev].stamp[s] > g_chain_dev[dev].stamp[best]))
            best = s;
    if (best >= 0) *mhz = (float)((double)ctl[best * 16 + 11] / (double)ctl[best * 16 + 12] * 100.0);
    return hipSuccess;
}

}  // namespace ohip
