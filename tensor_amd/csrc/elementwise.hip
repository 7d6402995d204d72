// Bandwidth-bound elementwise kernels of the int8 path: quantize, dequantize, requantize, repack.
//
// One thread owns V consecutive channels of one pixel (V = the wider of the two packs involved), so that
// the packed side(s) move as 8/16/32-byte vectors and an unpacked side is read/written as V planes, each
// coalesced along the pixel index. No LDS: every byte is touched once.
#include "common.hpp"

namespace ohip {

template <typename T, int P, int V>
struct Access {
    static constexpr int CH = (P == 1) ? 1 : (P < V ? P : V);  // contiguous elements per chunk
    typedef T vec_t __attribute__((ext_vector_type(CH)));

    __device__ static __forceinline__ void load(const T* base, int n, int c0, int pix, int C, int HW, T (&v)[V]) {
        if constexpr (P == 1) {
            const T* p = base + ((size_t)n * C + c0) * HW + pix;
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = p[(size_t)j * HW];
        } else {
#pragma unroll
            for (int j = 0; j < V; j += CH) {
                const T* p = base + elem_offset(P, n, c0 + j, pix, C, HW);
                vec_t t = *reinterpret_cast<const vec_t*>(p);
#pragma unroll
                for (int i = 0; i < CH; ++i) v[j + i] = t[i];
            }
        }
    }

    __device__ static __forceinline__ void store(T* base, int n, int c0, int pix, int C, int HW, const T (&v)[V]) {
        if constexpr (P == 1) {
            T* p = base + ((size_t)n * C + c0) * HW + pix;
#pragma unroll
            for (int j = 0; j < V; ++j) p[(size_t)j * HW] = v[j];
        } else {
#pragma unroll
            for (int j = 0; j < V; j += CH) {
                T* p = base + elem_offset(P, n, c0 + j, pix, C, HW);
                vec_t t;
#pragma unroll
                for (int i = 0; i < CH; ++i) t[i] = v[j + i];
                *reinterpret_cast<vec_t*>(p) = t;
            }
        }
    }
};

struct QuantOp {
    const float* scales;  // null: `scale` for every channel
    int n_scales;
    int round_mode;
    float scale;
    template <int V>
    __device__ __forceinline__ void operator()(const float (&in)[V], int8_t (&out)[V], int c0) const {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float s = scales == nullptr ? scale : (n_scales == 1 ? scales[0] : scales[c0 + j]);
            out[j] = (int8_t)float2int8_rt(__fmul_rn(in[j], s), round_mode);
        }
    }
};

struct DequantOp {
    const float* scale;
    int n_scale;
    const float* bias;
    int n_bias;
    template <int V>
    __device__ __forceinline__ void operator()(const int32_t (&in)[V], float (&out)[V], int c0) const {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float s = n_scale == 1 ? scale[0] : scale[c0 + j];
            float b = n_bias == 0 ? 0.f : (n_bias == 1 ? bias[0] : bias[c0 + j]);
            out[j] = dequant_rt(in[j], s, b, n_bias != 0);
        }
    }
};

struct RequantOp {
    const float* scale_in;
    int n_scale_in;
    const float* scale_out;
    int n_scale_out;
    const float* bias;
    int n_bias;
    int act;
    float act_p0;
    int round_mode;
    template <int V>
    __device__ __forceinline__ void operator()(const int32_t (&in)[V], int8_t (&out)[V], int c0) const {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float si = n_scale_in == 1 ? scale_in[0] : scale_in[c0 + j];
            float so = n_scale_out == 1 ? scale_out[0] : scale_out[c0 + j];
            float b = n_bias == 0 ? 0.f : (n_bias == 1 ? bias[0] : bias[c0 + j]);
            out[j] = (int8_t)requant_rt(in[j], si, b, n_bias != 0, act, act_p0, so, round_mode);
        }
    }
};

template <typename T>
struct CopyOp {
    template <int V>
    __device__ __forceinline__ void operator()(const T (&in)[V], T (&out)[V], int) const {
#pragma unroll
        for (int j = 0; j < V; ++j) out[j] = in[j];
    }
};

template <typename TI, typename TO, int SP, int DP, int V, class Op>
__global__ void __launch_bounds__(256) ew_kernel(const TI* __restrict__ src, TO* __restrict__ dst, int N, int C, int HW,
                                                 Op op) {
    // 32-bit indices (the C ABI refuses tensors of 2^31 elements or more): 64-bit divisions would cost more vector
    // instructions than the operation itself
    const unsigned cv_count = (unsigned)(C / V);
    const unsigned total = (unsigned)N * cv_count * (unsigned)HW;
    for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const unsigned r = idx / (unsigned)HW;
        const int pix = (int)(idx - r * (unsigned)HW);
        const int n = (int)(r / cv_count);
        const int cv = (int)(r - (unsigned)n * cv_count);
        TI in[V];
        TO out[V];
        Access<TI, SP, V>::load(src, n, cv * V, pix, C, HW, in);
        op.template operator()<V>(in, out, cv * V);
        Access<TO, DP, V>::store(dst, n, cv * V, pix, C, HW, out);
    }
}

template <typename TI, typename TO, int SP, int DP, class Op>
static hipError_t launch_ew(const TI* src, TO* dst, int N, int C, int HW, Op op, hipStream_t stream) {
    constexpr int V = SP > DP ? SP : DP;
    const size_t total = (size_t)N * (C / V) * HW;
    if (total == 0) return hipSuccess;
    size_t blocks = (total + 255) / 256;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    hipLaunchKernelGGL((ew_kernel<TI, TO, SP, DP, V, Op>), dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, N, C,
                       HW, op);
    return hipGetLastError();
}

// dispatch on (src pack, dst pack) among {1,4,8}; packs that do not divide C never reach here
template <typename TI, typename TO, class Op>
hipError_t dispatch_ew(const TI* src, int sp, TO* dst, int dp, int N, int C, int HW, Op op, hipStream_t stream) {
#define OHIP_CASE(SP, DP) \
    if (sp == SP && dp == DP) return launch_ew<TI, TO, SP, DP, Op>(src, dst, N, C, HW, op, stream);
    OHIP_CASE(1, 1)
    OHIP_CASE(1, 4)
    OHIP_CASE(1, 8)
    OHIP_CASE(4, 1)
    OHIP_CASE(4, 4)
    OHIP_CASE(4, 8)
    OHIP_CASE(8, 1)
    OHIP_CASE(8, 4)
    OHIP_CASE(8, 8)
#undef OHIP_CASE
    return hipErrorInvalidValue;
}

// [N, C, HW] in any pack dividing C (fp32, quantized on the way, or int8) -> Byte8 with the channel count padded with
// zeros to Cp = a multiple of 8: lets a convolution whose C is not a multiple of 8 (an RGB stem) use the MFMA path.
template <typename T>
__global__ void __launch_bounds__(256) pad_pack8_kernel(const T* __restrict__ src, int sp, int8_t* __restrict__ dst, int N,
                                                        int C, int Cp, int HW, const float* __restrict__ scale,
                                                        int round_mode) {
    const unsigned total = (unsigned)N * (unsigned)(Cp / 8) * (unsigned)HW;
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const unsigned r = idx / (unsigned)HW;
    const int pix = (int)(idx - r * (unsigned)HW);
    const int n = (int)(r / (unsigned)(Cp / 8));
    const int o = (int)(r - (unsigned)n * (unsigned)(Cp / 8));
    int q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int c = o * 8 + e;
        q[e] = 0;
        if (c < C) {
            const T v = src[elem_offset(sp, n, c, pix, C, HW)];
            if constexpr (sizeof(T) == 4) q[e] = float2int8_rt(__fmul_rn((float)v, scale[0]), round_mode);
            else q[e] = (int)v;
        }
    }
    ohip_v2i pk;
    pk[0] = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | (q[3] << 24);
    pk[1] = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | (q[7] << 24);
    reinterpret_cast<ohip_v2i*>(dst)[idx] = pk;
}

hipError_t run_pad_pack8(const void* src, bool src_is_float, int sp, int8_t* dst, int N, int C, int Cp, int HW,
                         const float* scale, int round_mode, hipStream_t stream) {
    const size_t total = (size_t)N * (Cp / 8) * HW;
    if (total == 0) return hipSuccess;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (src_is_float)
        hipLaunchKernelGGL(pad_pack8_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)src, sp, dst, N, C, Cp,
                           HW, scale, round_mode);
    else
        hipLaunchKernelGGL(pad_pack8_kernel<int8_t>, dim3(blocks), dim3(256), 0, stream, (const int8_t*)src, sp, dst, N, C,
                           Cp, HW, scale, round_mode);
    return hipGetLastError();
}

hipError_t run_quantize(const float* src, int sp, int8_t* dst, int dp, int N, int C, int HW, const float* scales,
                        int n_scales, int round_mode, hipStream_t stream) {
    QuantOp op{scales, n_scales, round_mode, 0.f};
    return dispatch_ew<float, int8_t, QuantOp>(src, sp, dst, dp, N, C, HW, op, stream);
}

hipError_t run_quantize_by(const float* src, int sp, int8_t* dst, int dp, int N, int C, int HW, float scale, int round_mode,
                           hipStream_t stream) {
    QuantOp op{nullptr, 1, round_mode, scale};
    return dispatch_ew<float, int8_t, QuantOp>(src, sp, dst, dp, N, C, HW, op, stream);
}

hipError_t run_dequantize(const int32_t* src, int sp, float* dst, int dp, int N, int C, int HW, const float* scale,
                          int n_scale, const float* bias, int n_bias, hipStream_t stream) {
    DequantOp op{scale, n_scale, bias, n_bias};
    return dispatch_ew<int32_t, float, DequantOp>(src, sp, dst, dp, N, C, HW, op, stream);
}

hipError_t run_requantize(const int32_t* src, int sp, int8_t* dst, int dp, int N, int C, int HW, const float* scale_in,
                          int n_scale_in, const float* scale_out, int n_scale_out, const float* bias, int n_bias,
                          int act, float act_p0, int round_mode, hipStream_t stream) {
    RequantOp op{scale_in, n_scale_in, scale_out, n_scale_out, bias, n_bias, act, act_p0, round_mode};
    return dispatch_ew<int32_t, int8_t, RequantOp>(src, sp, dst, dp, N, C, HW, op, stream);
}

hipError_t run_repack(const void* src, int sp, void* dst, int dp, int elem_bytes, int N, int C, int HW,
                      hipStream_t stream) {
    if (elem_bytes == 1)
        return dispatch_ew<int8_t, int8_t, CopyOp<int8_t>>((const int8_t*)src, sp, (int8_t*)dst, dp, N, C, HW,
                                                           CopyOp<int8_t>{}, stream);
    return dispatch_ew<int32_t, int32_t, CopyOp<int32_t>>((const int32_t*)src, sp, (int32_t*)dst, dp, N, C, HW,
                                                          CopyOp<int32_t>{}, stream);
}

}  // namespace ohip
