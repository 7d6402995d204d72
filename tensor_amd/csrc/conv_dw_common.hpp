// Device helpers shared by the depthwise matrix-core kernels (conv_dw_mfma.hip) and the pointwise + depthwise launch
// (conv_xdw.hip): buffer descriptors, the out-of-range offset, the requantization of four accumulators into one dword.
#pragma once

#include "common.hpp"

namespace ohip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v4u_store __attribute__((__vector_size__(4 * sizeof(unsigned))));
typedef unsigned v2u_store __attribute__((__vector_size__(2 * sizeof(unsigned))));

constexpr unsigned DW_OOB = 0x80000000u;  // beyond any descriptor this file builds (tensors are kept below 2 GiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dw_rsrc(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// Requantize four accumulators into four saturated bytes of one dword.
// The activation clamp [0, hi] is applied AFTER scaling and rounding, on the packed int16 values, instead of on the
// float before them: x -> trunc(fl(fl(x * so) + half)) is monotone for so > 0, so clamping its argument to [0, hi]
// equals clamping its result to [trunc(0 + half), trunc(fl(fl(hi * so) + half))] = [0, qh], bit for bit; qh (capped at
// the int8 saturation bound 127) is computed once per wave by dw_clamp_pair. Without an activation there is no clamp.
__device__ __forceinline__ unsigned dw_clamp_pair(const Epilogue& ep, int so0, int so1) {
    const int q0 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, __int_as_float(so0)), ep.round_half), 127);
    const int q1 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, __int_as_float(so1)), ep.round_half), 127);
    return (unsigned)(q0 & 0xffff) | ((unsigned)q1 << 16);
}

template <bool NONNEG>
__device__ __forceinline__ unsigned dw_requant4(const Epilogue& ep, const v4i& acc, const v4i& si, const v4i& bi,
                                                const v4i& so, unsigned qh01, unsigned qh23) {
    int qv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = __fmaf_rn((float)acc[e], __int_as_float(si[e]), __int_as_float(bi[e]));
        if (!NONNEG && ep.lrelu) v = fmaxf(v, __fmul_rn(v, ep.act_p0));  // wave-uniform branch
        v = __fmul_rn(v, __int_as_float(so[e]));
        const float adj = NONNEG ? __fadd_rn(v, ep.round_half) : __fadd_rn(v, __builtin_copysignf(ep.round_half, v));
        // toward zero, saturating; NONNEG: to unsigned, which is also the activation's lower clamp
        if constexpr (NONNEG) qv[e] = (int)cvt_u32_floor0(adj);
        else qv[e] = (int)adj;
    }
    if constexpr (NONNEG) {
        typedef unsigned short ohip_v2us __attribute__((ext_vector_type(2)));
        ohip_v2us lo = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)qv[0], (unsigned)qv[1]));
        ohip_v2us hi = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)qv[2], (unsigned)qv[3]));
        lo = __builtin_elementwise_min(lo, __builtin_bit_cast(ohip_v2us, qh01));
        hi = __builtin_elementwise_min(hi, __builtin_bit_cast(ohip_v2us, qh23));
        return __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
    }
    ohip_v2s lo = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(qv[0], qv[1]));
    ohip_v2s hi = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(qv[2], qv[3]));
    if (NONNEG) {
        const ohip_v2s zero = {0, 0};
        lo = __builtin_elementwise_max(__builtin_elementwise_min(lo, __builtin_bit_cast(ohip_v2s, qh01)), zero);
        hi = __builtin_elementwise_max(__builtin_elementwise_min(hi, __builtin_bit_cast(ohip_v2s, qh23)), zero);
    } else {
        const ohip_v2s top = {127, 127}, bot = {-127, -127};
        lo = __builtin_elementwise_max(__builtin_elementwise_min(lo, top), bot);
        hi = __builtin_elementwise_max(__builtin_elementwise_min(hi, top), bot);
    }
    return __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
}

}  // namespace ohip
