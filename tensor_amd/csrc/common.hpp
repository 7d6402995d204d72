// Shared device/host helpers of the gfx950 int8 convolution library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/otter_hip_int8.h"

namespace ohip {

// ---------------------------------------------------------------------------------------------------
// layouts
// ---------------------------------------------------------------------------------------------------
__host__ __device__ inline int layout_pack(int layout) {
    switch (layout) {
    case OTTER_HIP_F32_P4:
    case OTTER_HIP_I32_P4:
        return 4;
    case OTTER_HIP_F32_P8:
    case OTTER_HIP_I8_P8:
    case OTTER_HIP_I32_P8:
        return 8;
    default:
        return 1;
    }
}

// 0 = f32, 1 = i8, 2 = i32
__host__ __device__ inline int layout_elem(int layout) {
    if (layout <= OTTER_HIP_F32_P8) return 0;
    if (layout <= OTTER_HIP_I8_P8) return 1;
    return 2;
}

__host__ __device__ inline int layout_elem_bytes(int layout) { return layout_elem(layout) == 1 ? 1 : 4; }

// element offset of (n, c, pix) in a tensor [N, C/p, HW, p]
__host__ __device__ inline size_t elem_offset(int p, int n, int c, int pix, int C, int HW) {
    return (((size_t)n * (C / p) + (c / p)) * HW + pix) * p + (c % p);
}

// ---------------------------------------------------------------------------------------------------
// epilogue arithmetic: bit-for-bit what the reference's x86 build evaluates
// ---------------------------------------------------------------------------------------------------

// float2int8_sse (Tensor/VecIntrinsic.hpp:71-95): trunc(v + copysign(0.5f, v)), saturate to [-127,127].
// float2int8 (Tensor/QuantizeX86.cpp:18-23): (int)round(v). Adding the largest float below 0.5 before
// truncating rounds half away from zero exactly for every finite float, so the two primitives differ only
// in the constant.
template <int ROUND>
__device__ __forceinline__ int float2int8(float v) {
    const float half = (ROUND == OTTER_HIP_ROUND_SSE) ? 0.5f : 0.49999997f;
    float adj = __fadd_rn(v, __builtin_copysignf(half, v));
    int i = (int)adj;  // v_cvt_i32_f32: toward zero, saturating
    return min(max(i, -127), 127);
}

__device__ __forceinline__ int float2int8_rt(float v, int round_mode) {
    const float half = (round_mode == OTTER_HIP_ROUND_SSE) ? 0.5f : 0.49999997f;
    float adj = __fadd_rn(v, __builtin_copysignf(half, v));
    int i = (int)adj;
    return min(max(i, -127), 127);
}

// activation_sse (Tensor/QuantizeX86.hpp:72-106) and the Relu / LRelu / Relu6 / Sigmoid layers that follow
// dequantize on the fp32 path (Tensor/ConvolutionLayer.cpp:838-843)
__device__ __forceinline__ float activate(float v, int act, float p0) {
    switch (act) {
    case 1:
        return fmaxf(v, 0.f);
    case 2:
        return v > 0.f ? v : __fmul_rn(v, p0);
    case 3:
        return fminf(fmaxf(v, 0.f), 6.f);
    case 4:
        return 1.f / (1.f + __expf(-v));
    default:
        return v;
    }
}

// v = acc*scale_in (+bias, single rounding: the reference build contracts it to vfmadd)
template <bool BIAS>
__device__ __forceinline__ float dequant(int acc, float si, float b) {
    return BIAS ? __fmaf_rn((float)acc, si, b) : __fmul_rn((float)acc, si);
}

__device__ __forceinline__ float dequant_rt(int acc, float si, float b, bool has_bias) {
    return has_bias ? __fmaf_rn((float)acc, si, b) : __fmul_rn((float)acc, si);
}

__device__ __forceinline__ int requant_rt(int acc, float si, float b, bool has_bias, int act, float p0, float so,
                                          int round_mode) {
    float v = dequant_rt(acc, si, b, has_bias);
    v = activate(v, act, p0);
    v = __fmul_rn(v, so);
    return float2int8_rt(v, round_mode);
}

// ---------------------------------------------------------------------------------------------------
// epilogue parameters shared by every convolution kernel
// ---------------------------------------------------------------------------------------------------
struct Epilogue {
    const float* scale_in;   // [Kpad]
    const float* bias;       // [Kpad] or nullptr
    const float* scale_out;  // [Kpad] (broadcast on the host when one value was given)
    int act;
    float act_p0;
    int round_mode;
    int out_kind;    // otter_hip_out_kind
    int out_layout;  // otter_hip_layout
};

struct ConvGeom {
    int N, C, H, W;        // input
    int K, OH, OW;         // output
    int kh, kw, sh, sw, ph, pw, dh, dw;
    int groups;
};

// ---------------------------------------------------------------------------------------------------
// Shared tail of the MFMA and depthwise kernels: one lane holds the int32 accumulators of 8 consecutive
// output channels ch0..ch0+7 (ch0 % 8 == 0) of one output pixel; apply the epilogue and store them in the
// requested layout. si/bi/so are the per-channel scale_in / bias / scale_out of those 8 channels.
// ---------------------------------------------------------------------------------------------------
typedef int ohip_v4i __attribute__((ext_vector_type(4)));
typedef int ohip_v2i __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void epilogue_store8(void* __restrict__ out, const Epilogue& ep, int n, int ch0, int pix,
                                                int K, int OHW, const int (&a8)[8], const float (&si)[8],
                                                const float (&bi)[8], const float (&so)[8]) {
    const int out_pack = layout_pack(ep.out_layout);
    const bool has_bias = ep.bias != nullptr;
    if (ep.out_kind == OTTER_HIP_OUT_I8) {
        int q[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = dequant_rt(a8[e], si[e], bi[e], has_bias);
            v = activate(v, ep.act, ep.act_p0);
            q[e] = float2int8_rt(__fmul_rn(v, so[e]), ep.round_mode);
        }
        int8_t* o = (int8_t*)out;
        if (out_pack == 8) {
            ohip_v2i pk;
            pk[0] = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | ((q[3] & 0xff) << 24);
            pk[1] = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | ((q[7] & 0xff) << 24);
            *reinterpret_cast<ohip_v2i*>(o + elem_offset(8, n, ch0, pix, K, OHW)) = pk;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (ch0 + e < K) o[elem_offset(1, n, ch0 + e, pix, K, OHW)] = (int8_t)q[e];
        }
    } else {
        int r8[8];
        if (ep.out_kind == OTTER_HIP_OUT_F32) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = dequant_rt(a8[e], si[e], bi[e], has_bias);
                r8[e] = __float_as_int(activate(v, ep.act, ep.act_p0));
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) r8[e] = a8[e];
        }
        int* o = (int*)out;
        if (out_pack == 8) {
            int* p = o + elem_offset(8, n, ch0, pix, K, OHW);
            *reinterpret_cast<ohip_v4i*>(p) = ohip_v4i{r8[0], r8[1], r8[2], r8[3]};
            *reinterpret_cast<ohip_v4i*>(p + 4) = ohip_v4i{r8[4], r8[5], r8[6], r8[7]};
        } else if (out_pack == 4) {
            *reinterpret_cast<ohip_v4i*>(o + elem_offset(4, n, ch0, pix, K, OHW)) =
                ohip_v4i{r8[0], r8[1], r8[2], r8[3]};
            if (ch0 + 4 < K)
                *reinterpret_cast<ohip_v4i*>(o + elem_offset(4, n, ch0 + 4, pix, K, OHW)) =
                    ohip_v4i{r8[4], r8[5], r8[6], r8[7]};
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (ch0 + e < K) o[elem_offset(1, n, ch0 + e, pix, K, OHW)] = r8[e];
        }
    }
}

}  // namespace ohip
