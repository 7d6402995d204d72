// fp32 layout glue between the convolutions of a detection backbone (the layers the reference's int8 model files
// put around their convolutions): channel-range copy (Concat / Crop), channel shuffle, max pooling, 2-D upsampling.
// Every kernel takes any of the fp32 activation layouts on either side (elempack 1, 4 or 8: memory order
// n, c/p, h, w, c%p) and is a pure gather: one thread per destination element (or per group of four where source
// and destination packs line up), enumerated in destination memory order so that the writes are contiguous.
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

__device__ __forceinline__ size_t packed_off(int n, int c, int y, int x, int C, int H, int W, int p) {
    return ((((size_t)n * (C / p) + c / p) * H + y) * W + x) * p + c % p;
}

// destination memory order restricted to a channel range that starts and ends on a pack boundary:
// linear index -> (n, c, y, x)
struct DstIndex {
    int n, c, y, x;
};
// (32-bit arithmetic throughout: the C ABI refuses tensors of 2^31 elements or more)
__device__ __forceinline__ DstIndex dst_index(unsigned i, int c0, int cnt, int H, int W, int p) {
    DstIndex d;
    unsigned r = i / (unsigned)p;
    const int e = (int)(i - r * (unsigned)p);
    unsigned t = r / (unsigned)W;
    d.x = (int)(r - t * (unsigned)W);
    r = t / (unsigned)H;
    d.y = (int)(t - r * (unsigned)H);
    const unsigned packs = (unsigned)(cnt / p);
    t = r / packs;
    d.c = c0 + (int)(r - t * packs) * p + e;
    d.n = (int)t;
    return d;
}

// dst[:, cd0 : cd0+cnt] = src[:, cs0 : cs0+cnt]   (Tensor/ConcatLayer.cpp:54-67 one input at a time;
// Tensor/CropLayer.cpp:69-75 with axis 1). ALIGNED: cd0 and cnt are multiples of the destination pack.
template <bool ALIGNED>
__global__ void __launch_bounds__(256) copy_channels_kernel(const float* __restrict__ src, int Cs, int ps, int cs0,
                                                            float* __restrict__ dst, int Cd, int pd, int cd0, int cnt,
                                                            int N, int H, int W, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    DstIndex d;
    if (ALIGNED) {
        d = dst_index(i, cd0, cnt, H, W, pd);
    } else {  // channel-major enumeration; the writes of a packed destination are strided then
        unsigned r = i / (unsigned)W;
        d.x = (int)(i - r * (unsigned)W);
        unsigned t = r / (unsigned)H;
        d.y = (int)(r - t * (unsigned)H);
        r = t / (unsigned)cnt;
        d.c = cd0 + (int)(t - r * (unsigned)cnt);
        d.n = (int)r;
    }
    dst[packed_off(d.n, d.c, d.y, d.x, Cd, H, W, pd)] = src[packed_off(d.n, d.c - cd0 + cs0, d.y, d.x, Cs, H, W, ps)];
}

// same, four floats per thread: both packs are multiples of 4, the source offset is a multiple of 4 and the
// destination range starts and ends on a destination pack boundary
// With q: also the Byte8 quantization of the copied channels, q = float2int8(v * scale), at their place in a blob of Cd
// channels (Cd % 8 == 0): what an int8 convolution reading dst would compute first.
__global__ void __launch_bounds__(256) copy_channels4_kernel(const float* __restrict__ src, int Cs, int ps, int cs0,
                                                             float* __restrict__ dst, int Cd, int pd, int cd0, int cnt,
                                                             int N, int H, int W, unsigned total4, int8_t* __restrict__ qdst,
                                                             float scale, float half) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total4) return;
    // quads of the destination range in memory order: (n, pack, y, x, quad within the pack)
    const unsigned qd = (unsigned)(pd / 4);
    unsigned r = i / qd;
    const int q = (int)(i - r * qd);
    unsigned t = r / (unsigned)W;
    const int x = (int)(r - t * (unsigned)W);
    r = t / (unsigned)H;
    const int y = (int)(t - r * (unsigned)H);
    const unsigned packs = (unsigned)(cnt / pd);
    t = r / packs;
    const int c = cd0 + (int)(r - t * packs) * pd + 4 * q;
    const int n = (int)t;
    const float4 v = *reinterpret_cast<const float4*>(src + packed_off(n, c - cd0 + cs0, y, x, Cs, H, W, ps));
    *reinterpret_cast<float4*>(dst + packed_off(n, c, y, x, Cd, H, W, pd)) = v;
    if (qdst != nullptr) {  // uniform
        const float f[4] = {v.x, v.y, v.z, v.w};
        unsigned pk = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float t = __fmul_rn(f[e], scale);
            const int k = (int)__fadd_rn(t, __builtin_copysignf(half, t));
            pk |= (unsigned)(min(max(k, -127), 127) & 0xff) << (8 * e);
        }
        *reinterpret_cast<unsigned*>(qdst + packed_off(n, c, y, x, Cd, H, W, 8)) = pk;
    }
}

// A whole Concat over channels in one launch: up to CONCAT_MAX packed fp32 sources, every channel count a multiple of
// 4, into a packed destination; one thread per channel quad of one destination pixel, in destination memory order.
// With qdst also the Byte8 quantization of the result (Cd % 8 == 0), as in copy_channels4_kernel.
__global__ void __launch_bounds__(256) concat_channels4_kernel(ConcatSources srcs, float* __restrict__ dst, int Cd, int pd,
                                                               int H, int W, unsigned total4, int8_t* __restrict__ qdst,
                                                               float scale, float half) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total4) return;
    const unsigned qd = (unsigned)(pd / 4);
    unsigned r = i / qd;
    const int q = (int)(i - r * qd);
    unsigned t = r / (unsigned)W;
    const int x = (int)(r - t * (unsigned)W);
    r = t / (unsigned)H;
    const int y = (int)(t - r * (unsigned)H);
    const unsigned packs = (unsigned)(Cd / pd);
    t = r / packs;
    const int c = (int)(r - t * packs) * pd + 4 * q;
    const int n = (int)t;
    int k = 0;  // the source that holds destination channel c
#pragma unroll
    for (int j = 1; j < CONCAT_MAX; ++j)
        if (j < srcs.count && c >= srcs.first[j]) k = j;
    const float4 v = *reinterpret_cast<const float4*>(srcs.ptr[k] +
                                                      packed_off(n, c - srcs.first[k], y, x, srcs.channels[k], H, W, srcs.pack[k]));
    *reinterpret_cast<float4*>(dst + packed_off(n, c, y, x, Cd, H, W, pd)) = v;
    if (qdst != nullptr) {  // uniform
        const float f[4] = {v.x, v.y, v.z, v.w};
        unsigned pk = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float tt = __fmul_rn(f[e], scale);
            const int kk = (int)__fadd_rn(tt, __builtin_copysignf(half, tt));
            pk |= (unsigned)(min(max(kk, -127), 127) & 0xff) << (8 * e);
        }
        *reinterpret_cast<unsigned*>(qdst + packed_off(n, c, y, x, Cd, H, W, 8)) = pk;
    }
}

hipError_t run_concat_channels(const ConcatSources& srcs, float* dst, int Cd, int pd, int N, int H, int W, int8_t* q,
                               float scale, int round_mode, hipStream_t stream) {
    const size_t total4 = (size_t)N * Cd * H * W / 4;
    if (total4 == 0) return hipSuccess;
    hipLaunchKernelGGL(concat_channels4_kernel, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, stream, srcs, dst, Cd, pd,
                       H, W, (unsigned)total4, q, scale, round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f);
    return hipGetLastError();
}

bool copy_channels_moves_quads(int ps, int cs0, int pd, int cd0, int cnt) {
    return cd0 % pd == 0 && cnt % pd == 0 && ps % 4 == 0 && pd % 4 == 0 && cs0 % 4 == 0;
}

hipError_t run_copy_channels(const float* src, int Cs, int ps, int cs0, float* dst, int Cd, int pd, int cd0, int cnt, int N,
                             int H, int W, hipStream_t stream, int8_t* q, float scale, int round_mode) {
    const size_t total = (size_t)N * cnt * H * W;
    if (total == 0) return hipSuccess;
    const bool whole = cd0 % pd == 0 && cnt % pd == 0;
    if (q != nullptr && !copy_channels_moves_quads(ps, cs0, pd, cd0, cnt)) return hipErrorInvalidValue;
    if (copy_channels_moves_quads(ps, cs0, pd, cd0, cnt)) {
        const size_t total4 = total / 4;
        hipLaunchKernelGGL(copy_channels4_kernel, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, stream, src, Cs, ps,
                           cs0, dst, Cd, pd, cd0, cnt, N, H, W, (unsigned)total4, q, scale,
                           round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f);
    } else if (whole) {
        hipLaunchKernelGGL(copy_channels_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, Cs,
                           ps, cs0, dst, Cd, pd, cd0, cnt, N, H, W, (unsigned)total);
    } else {
        hipLaunchKernelGGL(copy_channels_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, Cs,
                           ps, cs0, dst, Cd, pd, cd0, cnt, N, H, W, (unsigned)total);
    }
    return hipGetLastError();
}

// Tensor/ChannelShuffleKernel.cpp:19-55: input seen as [n, g, C/g, ...], output as [n, C/g, g, ...]
__global__ void __launch_bounds__(256) channel_shuffle_kernel(const float* __restrict__ src, int ps, float* __restrict__ dst,
                                                              int pd, int N, int C, int H, int W, int groups, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const DstIndex d = dst_index(i, 0, C, H, W, pd);
    const int cpg = C / groups;
    const int cs = (d.c % groups) * cpg + d.c / groups;
    dst[i] = src[packed_off(d.n, cs, d.y, d.x, C, H, W, ps)];
}

// groups == 2 on elempack 8 (the ShuffleNetV2 block of the detection model): output pack q interleaves source channels
// 4q..4q+3 of the first half with the same four of the second half -- two 16-byte reads, two 16-byte writes per pixel
// qdst (or null): also the Byte8 quantization of the shuffled blob, for int8 convolutions that read it next
__global__ void __launch_bounds__(256) channel_shuffle2_p8_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                  int C, int HW, unsigned total, int8_t* __restrict__ qdst,
                                                                  float scale, float half_ulp) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;  // (n, output pack, pixel)
    if (i >= total) return;
    const unsigned r = i / (unsigned)HW;
    const int px = (int)(i - r * (unsigned)HW);
    const unsigned packs = (unsigned)(C / 8);
    const size_t n = r / packs;
    const int q = (int)(r - (unsigned)n * packs);
    const int half = C / 2;
    const int c0 = 4 * q, c1 = half + 4 * q;  // first source channel of each half
    const float* base = src + n * (size_t)C * HW;
    const float4 a = *reinterpret_cast<const float4*>(base + ((size_t)(c0 / 8) * HW + px) * 8 + c0 % 8);
    const float4 b = *reinterpret_cast<const float4*>(base + ((size_t)(c1 / 8) * HW + px) * 8 + c1 % 8);
    float4* o = reinterpret_cast<float4*>(dst + (n * (size_t)C * HW) + ((size_t)q * HW + px) * 8);
    o[0] = make_float4(a.x, b.x, a.y, b.y);
    o[1] = make_float4(a.z, b.z, a.w, b.w);
    if (qdst != nullptr) {  // uniform
        const float f[8] = {a.x, b.x, a.y, b.y, a.z, b.z, a.w, b.w};
        int v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float t = __fmul_rn(f[e], scale);
            const int k = (int)__fadd_rn(t, __builtin_copysignf(half_ulp, t));
            v[e] = min(max(k, -127), 127) & 0xff;
        }
        ohip_v2i pk;
        pk[0] = v[0] | (v[1] << 8) | (v[2] << 16) | (v[3] << 24);
        pk[1] = v[4] | (v[5] << 8) | (v[6] << 16) | (v[7] << 24);
        reinterpret_cast<ohip_v2i*>(qdst)[i] = pk;  // same (n, pack, pixel) order as dst
    }
}

// The ShuffleNetV2 unit tail in one pass: Concat(a, b) -> ChannelShuffle(2 groups) -> the two half Crops. With Ch channels
// in a and in b, the shuffled blob alternates a[j], b[j]; its first Ch channels are output c1, the rest c2. All four
// outputs in elempack 8, inputs in elempack 4 or 8 each; one thread per (image, pack of the shuffled blob, pixel).
// q2 (optional): the Byte8 quantization of c2 with `scale`, for an int8 convolution that reads c2 next.
__global__ void __launch_bounds__(256) shuffle2_split_p8_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                float* __restrict__ c1, float* __restrict__ c2,
                                                                int8_t* __restrict__ q2, float scale, float half, int Ch,
                                                                int HW, int pa, int pb, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const unsigned r = i / (unsigned)HW;
    const int px = (int)(i - r * (unsigned)HW);
    const unsigned packs = (unsigned)(Ch / 4);  // packs of the shuffled blob (2*Ch channels)
    const size_t n = r / packs;
    const int q = (int)(r - (unsigned)n * packs);
    const int cs = 4 * q;  // first source channel, in a and in b
    // a and b may each be Float4 or Float8 (pa, pb): four consecutive channels are contiguous in both
    const size_t sa = ((n * (size_t)(Ch / pa) + cs / pa) * HW + px) * pa + cs % pa;
    const size_t sb = ((n * (size_t)(Ch / pb) + cs / pb) * HW + px) * pb + cs % pb;
    const float4 x = *reinterpret_cast<const float4*>(a + sa), y = *reinterpret_cast<const float4*>(b + sb);
    const int half_packs = Ch / 8;
    float* dst = q < half_packs ? c1 : c2;
    const int qd = q < half_packs ? q : q - half_packs;
    float4* o = reinterpret_cast<float4*>(dst + (n * (size_t)half_packs + qd) * HW * 8 + (size_t)px * 8);
    o[0] = make_float4(x.x, y.x, x.y, y.y);
    o[1] = make_float4(x.z, y.z, x.w, y.w);
    if (q2 != nullptr && q >= half_packs) {
        const float v[8] = {x.x, y.x, x.y, y.y, x.z, y.z, x.w, y.w};
        int k[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float t = __fmul_rn(v[e], scale);
            k[e] = min(max((int)__fadd_rn(t, __builtin_copysignf(half, t)), -127), 127) & 0xff;
        }
        ohip_v2i pk;
        pk[0] = k[0] | (k[1] << 8) | (k[2] << 16) | (k[3] << 24);
        pk[1] = k[4] | (k[5] << 8) | (k[6] << 16) | (k[7] << 24);
        *reinterpret_cast<ohip_v2i*>(q2 + (n * (size_t)half_packs + qd) * HW * 8 + (size_t)px * 8) = pk;
    }
}

hipError_t run_shuffle2_split(const float* a, int pa, const float* b, int pb, float* c1, float* c2, int8_t* q2, float scale,
                              int round_mode, int N, int Ch, int HW, hipStream_t stream) {
    const size_t total = (size_t)N * (Ch / 4) * HW;
    if (total == 0) return hipSuccess;
    const float half = round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
    hipLaunchKernelGGL(shuffle2_split_p8_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a, b, c1, c2, q2,
                       scale, half, Ch, HW, pa, pb, (unsigned)total);
    return hipGetLastError();
}

bool channel_shuffle_can_quantize(int ps, int pd, int C, int groups) { return groups == 2 && ps == 8 && pd == 8 && C % 16 == 0; }

hipError_t run_channel_shuffle(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int groups,
                               hipStream_t stream, int8_t* q, float scale, int round_mode) {
    const size_t total = (size_t)N * C * H * W;
    if (total == 0) return hipSuccess;
    if (q != nullptr && !channel_shuffle_can_quantize(ps, pd, C, groups)) return hipErrorInvalidValue;
    if (channel_shuffle_can_quantize(ps, pd, C, groups)) {
        const size_t units = total / 8;
        hipLaunchKernelGGL(channel_shuffle2_p8_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, stream, src, dst, C,
                           H * W, (unsigned)units, q, scale, round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(channel_shuffle_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, ps, dst, pd,
                       N, C, H, W, groups, (unsigned)total);
    return hipGetLastError();
}

// Tensor/MaxPoolLayer.cpp:123-134 -> otter::max_pool2d: window over the padded input; a NaN in the window wins
// (Tensor/MaxPoolKernel.cpp, the comparison `(val > maxval) || isnan(val)`). pad_value is what a tap outside the
// image counts as: -inf in the reference's generic kernel, 0 in its packed 3x3 / 2x2 stride-2 kernels
// (Tensor/Pool.cpp:974, which pad the blob with zeros first).
__global__ void __launch_bounds__(256) maxpool_kernel(const float* __restrict__ src, int ps, float* __restrict__ dst, int pd,
                                                      int N, int C, int H, int W, int OH, int OW, int kh, int kw, int sh,
                                                      int sw, int ph, int pw, int dh, int dw, float pad_value, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const DstIndex d = dst_index(i, 0, C, OH, OW, pd);
    float m = -__builtin_inff();
    for (int u = 0; u < kh; ++u) {
        const int iy = d.y * sh - ph + u * dh;
        for (int v = 0; v < kw; ++v) {
            const int ix = d.x * sw - pw + v * dw;
            const bool inside = iy >= 0 && iy < H && ix >= 0 && ix < W;
            const float val = inside ? src[packed_off(d.n, d.c, iy, ix, C, H, W, ps)] : pad_value;
            if (val > m || val != val) m = val;
        }
    }
    dst[i] = m;
}

// the same window, four channels per thread: both layouts packed by a multiple of 4, so a channel quad of one pixel is one
// 16-byte access on either side; threads in destination memory order (n, pack, y, x, quad within the pack)
__global__ void __launch_bounds__(256) maxpool4_kernel(const float* __restrict__ src, int ps, float* __restrict__ dst, int pd,
                                                       int C, int H, int W, int OH, int OW, int kh, int kw, int sh, int sw,
                                                       int ph, int pw, int dh, int dw, float pad_value, unsigned total4) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total4) return;
    const unsigned qd = (unsigned)(pd / 4);
    unsigned r = i / qd;
    const int q = (int)(i - r * qd);
    unsigned t = r / (unsigned)OW;
    const int ox = (int)(r - t * (unsigned)OW);
    r = t / (unsigned)OH;
    const int oy = (int)(t - r * (unsigned)OH);
    const unsigned packs = (unsigned)(C / pd);
    t = r / packs;
    const int c = (int)(r - t * packs) * pd + 4 * q;
    const int n = (int)t;
    const float ninf = -__builtin_inff();
    float m[4] = {ninf, ninf, ninf, ninf};
    for (int u = 0; u < kh; ++u) {
        const int iy = oy * sh - ph + u * dh;
        for (int v = 0; v < kw; ++v) {
            const int ix = ox * sw - pw + v * dw;
            const bool inside = iy >= 0 && iy < H && ix >= 0 && ix < W;
            float4 val = make_float4(pad_value, pad_value, pad_value, pad_value);
            if (inside) val = *reinterpret_cast<const float4*>(src + packed_off(n, c, iy, ix, C, H, W, ps));
            const float f[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (f[e] > m[e] || f[e] != f[e]) m[e] = f[e];
        }
    }
    *reinterpret_cast<float4*>(dst + packed_off(n, c, oy, ox, C, OH, OW, pd)) = make_float4(m[0], m[1], m[2], m[3]);
}

hipError_t run_maxpool(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int OH, int OW, int kh,
                       int kw, int sh, int sw, int ph, int pw, int dh, int dw, float pad_value, hipStream_t stream) {
    const size_t total = (size_t)N * C * OH * OW;
    if (total == 0) return hipSuccess;
    if (ps % 4 == 0 && pd % 4 == 0) {
        const size_t total4 = total / 4;
        hipLaunchKernelGGL(maxpool4_kernel, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, stream, src, ps, dst, pd, C, H,
                           W, OH, OW, kh, kw, sh, sw, ph, pw, dh, dw, pad_value, (unsigned)total4);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(maxpool_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, ps, dst, pd, N, C, H,
                       W, OH, OW, kh, kw, sh, sw, ph, pw, dh, dw, pad_value, (unsigned)total);
    return hipGetLastError();
}

// Source index and weight of one output coordinate: Tensor/TensorInterpolation.cpp:16-45 (linear_coeffs), the
// coefficient computation in double precision, the clamp at both borders included.
__device__ __forceinline__ void linear_coeff(int in_size, int out_size, int d, int align_corner, int& s, float& f) {
    double scale = (double)in_size / out_size;
    if (align_corner) scale = (double)(in_size - 1) / (out_size - 1);
    f = (float)((d + 0.5) * scale - 0.5);
    if (align_corner) f = (float)(d * scale);
    s = (int)floorf(f);
    f -= (float)s;
    if (s < 0) s = 0, f = 0.f;
    if (s >= in_size - 1) s = in_size - 2, f = 1.f;
}

// mode 1 nearest (Tensor/TensorInterpolation.cpp:670-690: source = min(int(d * in/out), in-1), the ratio in fp32),
// mode 2 bilinear (Tensor/TensorInterpolation.cpp:161-272: rows = S0*a0 then fma(S1, a1, .); out = rows0*b0 then
// fma(rows1, b1, .)) -- the arithmetic of the reference's packed path, which is what its Net runs when the channel
// count is a multiple of 4.
__global__ void __launch_bounds__(256) upsample_kernel(const float* __restrict__ src, int ps, float* __restrict__ dst, int pd,
                                                       int N, int C, int H, int W, int OH, int OW, int mode,
                                                       int align_corner, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const DstIndex d = dst_index(i, 0, C, OH, OW, pd);
    if (mode == 1) {
        const float hs = (float)H / (float)OH, ws = (float)W / (float)OW;
        const int iy = min((int)(d.y * hs), H - 1), ix = min((int)(d.x * ws), W - 1);
        dst[i] = src[packed_off(d.n, d.c, iy, ix, C, H, W, ps)];
        return;
    }
    int sx, sy;
    float fx, fy;
    linear_coeff(W, OW, d.x, align_corner, sx, fx);
    linear_coeff(H, OH, d.y, align_corner, sy, fy);
    const float a0 = 1.f - fx, a1 = fx, b0 = 1.f - fy, b1 = fy;
    const float s00 = src[packed_off(d.n, d.c, sy, sx, C, H, W, ps)], s01 = src[packed_off(d.n, d.c, sy, sx + 1, C, H, W, ps)];
    const float s10 = src[packed_off(d.n, d.c, sy + 1, sx, C, H, W, ps)],
                s11 = src[packed_off(d.n, d.c, sy + 1, sx + 1, C, H, W, ps)];
    const float r0 = __fmaf_rn(s01, a1, __fmul_rn(s00, a0));
    const float r1 = __fmaf_rn(s11, a1, __fmul_rn(s10, a0));
    dst[i] = __fmaf_rn(r1, b1, __fmul_rn(r0, b0));
}

// the same arithmetic, four channels per thread (both layouts packed by a multiple of 4): the coefficients of a pixel are
// computed once per channel quad, every tap is one 16-byte read
__global__ void __launch_bounds__(256) upsample4_kernel(const float* __restrict__ src, int ps, float* __restrict__ dst, int pd,
                                                        int C, int H, int W, int OH, int OW, int mode, int align_corner,
                                                        unsigned total4) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total4) return;
    const unsigned qd = (unsigned)(pd / 4);
    unsigned r = i / qd;
    const int q = (int)(i - r * qd);
    unsigned t = r / (unsigned)OW;
    const int ox = (int)(r - t * (unsigned)OW);
    r = t / (unsigned)OH;
    const int oy = (int)(t - r * (unsigned)OH);
    const unsigned packs = (unsigned)(C / pd);
    t = r / packs;
    const int c = (int)(r - t * packs) * pd + 4 * q;
    const int n = (int)t;
    auto at = [&](int y, int x) { return *reinterpret_cast<const float4*>(src + packed_off(n, c, y, x, C, H, W, ps)); };
    float4* out = reinterpret_cast<float4*>(dst + packed_off(n, c, oy, ox, C, OH, OW, pd));
    if (mode == 1) {
        const float hs = (float)H / (float)OH, ws = (float)W / (float)OW;
        *out = at(min((int)(oy * hs), H - 1), min((int)(ox * ws), W - 1));
        return;
    }
    int sx, sy;
    float fx, fy;
    linear_coeff(W, OW, ox, align_corner, sx, fx);
    linear_coeff(H, OH, oy, align_corner, sy, fy);
    const float a0 = 1.f - fx, a1 = fx, b0 = 1.f - fy, b1 = fy;
    const float4 s00 = at(sy, sx), s01 = at(sy, sx + 1), s10 = at(sy + 1, sx), s11 = at(sy + 1, sx + 1);
    auto mix = [&](float v00, float v01, float v10, float v11) {
        const float r0 = __fmaf_rn(v01, a1, __fmul_rn(v00, a0));
        const float r1 = __fmaf_rn(v11, a1, __fmul_rn(v10, a0));
        return __fmaf_rn(r1, b1, __fmul_rn(r0, b0));
    };
    *out = make_float4(mix(s00.x, s01.x, s10.x, s11.x), mix(s00.y, s01.y, s10.y, s11.y), mix(s00.z, s01.z, s10.z, s11.z),
                       mix(s00.w, s01.w, s10.w, s11.w));
}

hipError_t run_upsample(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int OH, int OW, int mode,
                        int align_corner, hipStream_t stream) {
    const size_t total = (size_t)N * C * OH * OW;
    if (total == 0) return hipSuccess;
    if (ps % 4 == 0 && pd % 4 == 0 && H > 1 && W > 1) {
        const size_t total4 = total / 4;
        hipLaunchKernelGGL(upsample4_kernel, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, stream, src, ps, dst, pd, C, H,
                           W, OH, OW, mode, align_corner, (unsigned)total4);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(upsample_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, ps, dst, pd, N, C, H,
                       W, OH, OW, mode, align_corner, (unsigned)total);
    return hipGetLastError();
}

}  // namespace ohip
