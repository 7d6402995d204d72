// fp32 glue of an int8 network between its convolution layers: element-wise add (residual connections), ReLU-type
// activations in place, global average pooling and the final inner product. All are bandwidth- or latency-bound
// and tiny next to the convolutions; they exist so that a whole network stays resident on the GPU.
#include "common.hpp"
#include "conv_igemm.hpp"

namespace ohip {

// out = a + b (Tensor/EltwiseLayer.cpp:48-80, operation sum); layouts must match, so it is a flat add
__global__ void __launch_bounds__(256) eltwise_add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          float* __restrict__ out, size_t n4, size_t n) {
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

// mean over H*W per (n, c); input in any fp32 layout, output [N, C] unpacked. One wave per (n, c).
__global__ void __launch_bounds__(256) global_avgpool_kernel(const float* __restrict__ x, int pack, int N, int C, int HW,
                                                             float* __restrict__ out) {
    const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (wave >= N * C) return;
    const int n = wave / C, c = wave % C;
    float s = 0.f;
    for (int i = lane; i < HW; i += 64) s += x[elem_offset(pack, n, c, i, C, HW)];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_down(s, o, 64);
    if (lane == 0) out[wave] = s / (float)HW;
}

// y[n][o] = sum_i x[n][i] * w[o][i] + b[o]   (Tensor/InnerProductLayer.cpp:176-, fp32). One wave per output.
__global__ void __launch_bounds__(256) inner_product_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ b, float* __restrict__ y, int N,
                                                            int IN, int OUT) {
    const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (wave >= N * OUT) return;
    const int n = wave / OUT, o = wave % OUT;
    float s = 0.f;
    for (int i = lane; i < IN; i += 64) s = __fmaf_rn(x[(size_t)n * IN + i], w[(size_t)o * IN + i], s);
#pragma unroll
    for (int k = 32; k > 0; k >>= 1) s += __shfl_down(s, k, 64);
    if (lane == 0) y[wave] = s + (b ? b[o] : 0.f);
}

hipError_t run_eltwise_add(const float* a, const float* b, float* out, size_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    const size_t n4 = n / 4;
    const size_t blocks = (n4 + 255) / 256 + (n4 == 0 ? 1 : 0);
    hipLaunchKernelGGL(eltwise_add_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, out, n4, n);
    return hipGetLastError();
}

hipError_t run_activation(float* x, size_t n, int act, float p0, hipStream_t stream) {
    if (n == 0 || act == 0) return hipSuccess;
    hipLaunchKernelGGL(activation_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, n, act, p0);
    return hipGetLastError();
}

hipError_t run_global_avgpool(const float* x, int pack, int N, int C, int HW, float* out, hipStream_t stream) {
    if (N * C == 0) return hipSuccess;
    hipLaunchKernelGGL(global_avgpool_kernel, dim3((N * C + 3) / 4), dim3(256), 0, stream, x, pack, N, C, HW, out);
    return hipGetLastError();
}

hipError_t run_inner_product(const float* x, const float* w, const float* b, float* y, int N, int IN, int OUT,
                             hipStream_t stream) {
    if (N * OUT == 0) return hipSuccess;
    hipLaunchKernelGGL(inner_product_kernel, dim3((N * OUT + 3) / 4), dim3(256), 0, stream, x, w, b, y, N, IN, OUT);
    return hipGetLastError();
}

}  // namespace ohip
