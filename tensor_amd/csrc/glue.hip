// fp32 glue of an int8 network between its convolution layers: element-wise add (residual connections), ReLU-type
// activations in place, global average pooling and the final inner product. All are bandwidth- or latency-bound
// and tiny next to the convolutions; they exist so that a whole network stays resident on the GPU.
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

// out = a + b (Tensor/EltwiseLayer.cpp:48-80, operation sum); layouts must match, so it is a flat add.
// `out` may be `a` (every element is read and written by one thread): no __restrict__ on the two.
__global__ void __launch_bounds__(256) eltwise_add_kernel(const float* a, const float* __restrict__ b, float* out, size_t n4,
                                                          size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) {
        const float4 x = reinterpret_cast<const float4*>(a)[i], y = reinterpret_cast<const float4*>(b)[i];
        reinterpret_cast<float4*>(out)[i] = make_float4(__fadd_rn(x.x, y.x), __fadd_rn(x.y, y.y), __fadd_rn(x.z, y.z),
                                                        __fadd_rn(x.w, y.w));
    }
    if (i == 0)
        for (size_t k = n4 * 4; k < n; ++k) out[k] = __fadd_rn(a[k], b[k]);
}

__global__ void __launch_bounds__(256) activation_kernel(float* __restrict__ x, size_t n, int act, float p0) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] = activate(x[i], act, p0);
}

// mean over H*W per (n, c); input in any fp32 layout, output [N, C] unpacked. One wave per (n, channel pack): a lane
// reads whole packs (4, 16 or 32 contiguous bytes per pixel), so a wave's reads are contiguous in every layout.
template <int P>
__global__ void __launch_bounds__(256) global_avgpool_kernel(const float* __restrict__ x, int N, int C, int HW,
                                                             float* __restrict__ out) {
    typedef float vec_t __attribute__((ext_vector_type(P)));
    const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    const int CP = C / P;
    if (wave >= N * CP) return;
    const int n = wave / CP, cp = wave % CP;
    const float* src = x + ((size_t)n * CP + cp) * HW * P;
    float s[P];
#pragma unroll
    for (int e = 0; e < P; ++e) s[e] = 0.f;
    for (int i = lane; i < HW; i += 64) {
        if constexpr (P == 1) {
            s[0] += src[i];
        } else {
            const vec_t v = *reinterpret_cast<const vec_t*>(src + (size_t)i * P);
#pragma unroll
            for (int e = 0; e < P; ++e) s[e] += v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < P; ++e) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) s[e] += __shfl_down(s[e], o, 64);
    }
    if (lane == 0) {
#pragma unroll
        for (int e = 0; e < P; ++e) out[(size_t)n * C + cp * P + e] = s[e] / (float)HW;
    }
}

// y[n][o] = sum_i x[n][i] * w[o][i] + b[o]   (Tensor/InnerProductLayer.cpp:176-, fp32).
// A workgroup owns IP_OB outputs x IP_NB images; its four waves split the reduction index, every lane keeps the
// IP_OB x IP_NB partial sums of its own indices in registers (each loaded weight is used IP_NB times, each input IP_OB
// times), and the 256 partial sums per result are added up through LDS at the end.
constexpr int IP_OB = 4, IP_NB = 8;
__global__ void __launch_bounds__(256) inner_product_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ b, float* __restrict__ y, int N,
                                                            int IN, int OUT) {
    __shared__ float part[IP_OB * IP_NB][257];
    const int o0 = blockIdx.x * IP_OB, n0 = blockIdx.y * IP_NB;
    const float* wr[IP_OB];
    const float* xr[IP_NB];
#pragma unroll
    for (int j = 0; j < IP_OB; ++j) wr[j] = w + (size_t)min(o0 + j, OUT - 1) * IN;  // clamped rows are computed, not stored
#pragma unroll
    for (int k = 0; k < IP_NB; ++k) xr[k] = x + (size_t)min(n0 + k, N - 1) * IN;
    float acc[IP_OB][IP_NB];
#pragma unroll
    for (int j = 0; j < IP_OB; ++j)
#pragma unroll
        for (int k = 0; k < IP_NB; ++k) acc[j][k] = 0.f;
    for (int i = threadIdx.x; i < IN; i += 256) {
        float wv[IP_OB], xv[IP_NB];
#pragma unroll
        for (int j = 0; j < IP_OB; ++j) wv[j] = wr[j][i];
#pragma unroll
        for (int k = 0; k < IP_NB; ++k) xv[k] = xr[k][i];
#pragma unroll
        for (int j = 0; j < IP_OB; ++j)
#pragma unroll
            for (int k = 0; k < IP_NB; ++k) acc[j][k] = __fmaf_rn(wv[j], xv[k], acc[j][k]);
    }
#pragma unroll
    for (int j = 0; j < IP_OB; ++j)
#pragma unroll
        for (int k = 0; k < IP_NB; ++k) part[j * IP_NB + k][threadIdx.x] = acc[j][k];
    __syncthreads();
    // four threads per result, 64 partial sums each
    const int r = threadIdx.x >> 2, q = threadIdx.x & 3;
    if (r >= IP_OB * IP_NB) return;  // whole waves: results 0..31 live in the first two
    float s = 0.f;
    for (int t = 0; t < 64; ++t) s += part[r][t * 4 + q];
    s += __shfl_xor(s, 1, 64);
    s += __shfl_xor(s, 2, 64);
    const int o = o0 + r / IP_NB, n = n0 + r % IP_NB;
    if (q == 0 && o < OUT && n < N) y[(size_t)n * OUT + o] = s + (b ? b[o] : 0.f);
}

hipError_t run_eltwise_add(const float* a, const float* b, float* out, size_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    const size_t n4 = n / 4;
    const size_t blocks = (n4 + 255) / 256 + (n4 == 0 ? 1 : 0);
    hipLaunchKernelGGL(eltwise_add_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, out, n4, n);
    return hipGetLastError();
}

// out = a + b and, in the same pass, the int8 blob a following int8 convolution would make of it
// (ConvolutionLayer::forward_int8 quantizes an fp32 bottom blob first, Tensor/ConvolutionLayer.cpp:770-775):
// q = float2int8(out * scale) into Byte8. One thread per (image, channel octet, pixel); P = elempack of a, b and out.
// `out` may be `a`.
template <int P>
__global__ void __launch_bounds__(256) eltwise_add_quantize_kernel(const float* a, const float* __restrict__ b, float* out,
                                                                   int8_t* __restrict__ q, int C8, int HW, float scale,
                                                                   float half, unsigned total) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const unsigned r = i / (unsigned)HW;
    const unsigned pix = i - r * (unsigned)HW;  // r = image * C8 + octet
    float s[8];
    if constexpr (P == 8) {
        const size_t o = (size_t)i * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float4 x = *reinterpret_cast<const float4*>(a + o + 4 * h), y = *reinterpret_cast<const float4*>(b + o + 4 * h);
            const float4 z = make_float4(__fadd_rn(x.x, y.x), __fadd_rn(x.y, y.y), __fadd_rn(x.z, y.z), __fadd_rn(x.w, y.w));
            *reinterpret_cast<float4*>(out + o + 4 * h) = z;
            s[4 * h] = z.x, s[4 * h + 1] = z.y, s[4 * h + 2] = z.z, s[4 * h + 3] = z.w;
        }
    } else {  // Float4: the octet's two packs are the planes 2r and 2r+1
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const size_t o = ((size_t)(2 * r + h) * HW + pix) * 4;
            const float4 x = *reinterpret_cast<const float4*>(a + o), y = *reinterpret_cast<const float4*>(b + o);
            const float4 z = make_float4(__fadd_rn(x.x, y.x), __fadd_rn(x.y, y.y), __fadd_rn(x.z, y.z), __fadd_rn(x.w, y.w));
            *reinterpret_cast<float4*>(out + o) = z;
            s[4 * h] = z.x, s[4 * h + 1] = z.y, s[4 * h + 2] = z.z, s[4 * h + 3] = z.w;
        }
    }
    int v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float t = __fmul_rn(s[e], scale);
        const int k = (int)__fadd_rn(t, __builtin_copysignf(half, t));
        v[e] = min(max(k, -127), 127) & 0xff;
    }
    ohip_v2i pk;
    pk[0] = v[0] | (v[1] << 8) | (v[2] << 16) | (v[3] << 24);
    pk[1] = v[4] | (v[5] << 8) | (v[6] << 16) | (v[7] << 24);
    reinterpret_cast<ohip_v2i*>(q)[i] = pk;
}

hipError_t run_eltwise_add_quantize(const float* a, const float* b, int pack, float* out, int8_t* q, int N, int C, int HW,
                                    float scale, int round_mode, hipStream_t stream) {
    const size_t total = (size_t)N * (C / 8) * HW;
    if (total == 0) return hipSuccess;
    const float half = round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (pack == 8)
        hipLaunchKernelGGL(eltwise_add_quantize_kernel<8>, grid, block, 0, stream, a, b, out, q, C / 8, HW, scale, half,
                           (unsigned)total);
    else
        hipLaunchKernelGGL(eltwise_add_quantize_kernel<4>, grid, block, 0, stream, a, b, out, q, C / 8, HW, scale, half,
                           (unsigned)total);
    return hipGetLastError();
}

hipError_t run_activation(float* x, size_t n, int act, float p0, hipStream_t stream) {
    if (n == 0 || act == 0) return hipSuccess;
    hipLaunchKernelGGL(activation_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, n, act, p0);
    return hipGetLastError();
}

hipError_t run_global_avgpool(const float* x, int pack, int N, int C, int HW, float* out, hipStream_t stream) {
    if (N * C == 0) return hipSuccess;
    const unsigned blocks = (unsigned)((N * (C / pack) + 3) / 4);
    if (pack == 8) hipLaunchKernelGGL(global_avgpool_kernel<8>, dim3(blocks), dim3(256), 0, stream, x, N, C, HW, out);
    else if (pack == 4) hipLaunchKernelGGL(global_avgpool_kernel<4>, dim3(blocks), dim3(256), 0, stream, x, N, C, HW, out);
    else if (pack == 1) hipLaunchKernelGGL(global_avgpool_kernel<1>, dim3(blocks), dim3(256), 0, stream, x, N, C, HW, out);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// The same product on the fp32 matrix cores, for the shapes of a classifier (a batch of up to a few hundred rows, IN a
// multiple of 16): the kernel above re-reads the weights once per 8 rows of x and multiplies on the vector ALU; here a
// workgroup multiplies 16 weight rows with 16 rows of x. v_mfma_f32_16x16x4f32: lane (i, kq)
// supplies A[i][kq] and B[kq][i]; with one 16-byte load per lane (4 consecutive inputs of weight row i / x row i) four
// instructions cover 16 inputs. The waves split the inputs and add their accumulators up through LDS.
typedef float ip_v4f __attribute__((ext_vector_type(4)));
constexpr int IPM_WAVES = 16;  // the inputs are dealt to 16 waves: a wave requests all its loads at once (one memory latency)
// A workgroup owns 16 outputs x 16 rows of x: enough workgroups to put every compute unit's memory pipeline to work
// (1000 outputs x 64 rows: 252 of them), each weight row read once per 16 rows of x.
// ALIGNED: both pointers are multiples of 16 bytes (one 16-byte load per operand); otherwise the same four floats come
// from four 4-byte loads -- the arithmetic, and so every bit of the result, is the same either way.
template <bool ALIGNED>
__global__ void __launch_bounds__(64 * IPM_WAVES) inner_product_mfma_kernel(const float* __restrict__ x,
                                                                            const float* __restrict__ w,
                                                                            const float* __restrict__ b, float* __restrict__ y,
                                                                            int N, int IN, int OUT) {
    __shared__ ip_v4f part[IPM_WAVES][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, kq = lane >> 4;
    const int o0 = blockIdx.x * 16, n0 = blockIdx.y * 16;
    const float* wr = w + (size_t)min(o0 + i, OUT - 1) * IN + 4 * kq;  // clamped rows are computed, not stored
    const float* xr = x + (size_t)min(n0 + i, N - 1) * IN + 4 * kq;
    ip_v4f acc = {0.f, 0.f, 0.f, 0.f};
    const int steps = IN / 16;
#pragma unroll 5
    for (int st = wave; st < steps; st += IPM_WAVES) {
        ip_v4f a, bv;
        if constexpr (ALIGNED) {
            a = *reinterpret_cast<const ip_v4f*>(wr + 16 * st);
            bv = *reinterpret_cast<const ip_v4f*>(xr + 16 * st);
        } else {
#pragma unroll
            for (int m = 0; m < 4; ++m) a[m] = wr[16 * st + m], bv[m] = xr[16 * st + m];
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[m], bv[m], acc, 0, 0, 0);
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave) return;
    // lane (i, kq) holds outputs o0 + 4 kq + r of x row n0 + i
    ip_v4f s = part[0][lane];
#pragma unroll
    for (int v = 1; v < IPM_WAVES; ++v) {
        const ip_v4f t = part[v][lane];
        s = ip_v4f{s[0] + t[0], s[1] + t[1], s[2] + t[2], s[3] + t[3]};
    }
    const int n = n0 + i;
    if (n < N) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int o = o0 + 4 * kq + r;
            if (o < OUT) y[(size_t)n * OUT + o] = s[r] + (b ? b[o] : 0.f);
        }
    }
}

hipError_t run_inner_product(const float* x, const float* w, const float* b, float* y, int N, int IN, int OUT,
                             hipStream_t stream) {
    if (N * OUT == 0) return hipSuccess;
    // The choice depends on the layer's shape only -- not on N (a row's result is then the same bits whatever batch it
    // sits in) and not on where the buffers lie (the two kernels add in different orders, so the same call must not give
    // different bits from one allocation to the next); alignment only picks how the matrix-core kernel loads.
    if (IN % 16 == 0 && IN >= 64) {
        const dim3 grid((OUT + 15) / 16, (N + 15) / 16), block(64 * IPM_WAVES);
        if ((((uintptr_t)x | (uintptr_t)w) & 15) == 0)
            hipLaunchKernelGGL(inner_product_mfma_kernel<true>, grid, block, 0, stream, x, w, b, y, N, IN, OUT);
        else
            hipLaunchKernelGGL(inner_product_mfma_kernel<false>, grid, block, 0, stream, x, w, b, y, N, IN, OUT);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(inner_product_kernel, dim3((OUT + IP_OB - 1) / IP_OB, (N + IP_NB - 1) / IP_NB), dim3(256), 0, stream,
                       x, w, b, y, N, IN, OUT);
    return hipGetLastError();
}

// The shader clock under matrix load: every wave runs int8 matrix instructions for `iters` rounds and brackets them with
// the shader-clock counter (s_memtime) and the constant 100 MHz counter (s_memrealtime); wave 0 of every workgroup
// writes its two differences. A workgroup per compute unit, four waves each (one per SIMD).
__global__ void __launch_bounds__(256) shader_clock_kernel(int iters, unsigned long long* __restrict__ out) {
    typedef int ck_v4i __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63;
    ck_v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane * 3, 1, 2, 3};
    ck_v4i acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[i], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = c1 - c0;
        out[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (acc[0][0] + acc[1][1] + acc[2][2] + acc[3][3] == 0x7fffffff) out[0] = 0;  // (keeps the loop)
}

hipError_t run_shader_clock(int blocks, int iters, unsigned long long* out, hipStream_t stream) {
    hipLaunchKernelGGL(shader_clock_kernel, dim3(blocks), dim3(256), 0, stream, iters, out);
    return hipGetLastError();
}

}  // namespace ohip
