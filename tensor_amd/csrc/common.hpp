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
    case 5:  // mish: reachable through the standalone requantize only (no option string of the layer selects it)
        return __fmul_rn(v, tanhf(logf(__expf(v) + 1.f)));
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
    // fast epilogues (activation none / ReLU / clip[0,6] as one clamp, rounding mode as one constant)
    float act_lo, act_hi;  // v = min(max(v, act_lo), act_hi)
    float round_half;      // 0.5f (ROUND_SSE) or 0.49999997f (ROUND_EXACT)
    bool so_positive;      // every output scale is finite and > 0 (lets the int8 epilogue clamp after rounding)
    bool lrelu;            // LeakyReLU with a slope in [0, 1]: v = max(v, v * act_p0), applied by the fast epilogues
    // fp32 output only: also write the Byte8 quantization of the result, q = float2int8(v * twin_scale), for an int8
    // convolution that reads this blob next (null: no twin). Honoured by the implicit-GEMM Float4 epilogue.
    int8_t* twin = nullptr;
    float twin_scale = 0.f, twin_half = 0.5f;
    // fp32 output only: a blob in the output's layout that is added to the activated result (the Eltwise sum of a
    // residual block; null: none). The twin, if any, is the quantization of the sum. Float4 epilogue only.
    const float* residual = nullptr;
};

// which epilogue code a kernel instance carries
enum {
    EPI_GENERIC = 0,
    EPI_I8_P8 = 1,
    EPI_F32_P4 = 2,
    EPI_I8_P8_NONNEG = 3,
    EPI_F32_P8 = 4,       // depthwise only
    EPI_F32_P4_FUSED = 5  // implicit GEMM only: EPI_F32_P4 plus the residual addend and / or the int8 twin
};

// The fast epilogues need: activation in {none, ReLU, clip, LeakyReLU with a slope in [0, 1]}, and (I8_P8) int8
// output in Byte8 with K % 8 == 0 or (F32_P4) fp32 output in Float4 with K % 4 == 0.
// LeakyReLU there is v = max(v, v * slope): equal to (v > 0 ? v : v * slope) for every v when 0 <= slope <= 1.
__host__ inline int pick_epilogue(const Epilogue& ep, int K) {
    const bool clamp_act = ep.act == 0 || ep.act == 1 || ep.act == 3 || (ep.act == 2 && ep.lrelu);
    if (clamp_act && ep.out_kind == OTTER_HIP_OUT_I8 && ep.out_layout == OTTER_HIP_I8_P8 && K % 8 == 0) {
        if (ep.act == 0 || ep.act == 2) return EPI_I8_P8;  // signed result: no clamp but the int8 range
        // after ReLU / clip the value to round is never negative; the fast path needs positive output scales
        return ep.so_positive ? EPI_I8_P8_NONNEG : EPI_GENERIC;
    }
    if (clamp_act && ep.out_kind == OTTER_HIP_OUT_F32 && ep.out_layout == OTTER_HIP_F32_P4 && K % 4 == 0) return EPI_F32_P4;
    return EPI_GENERIC;
}

struct ConvGeom {
    int N, C, H, W;        // input
    int K, OH, OW;         // output
    int kh, kw, sh, sw, ph, pw, dh, dw;
    int groups;
    // channels per image of the tensors in memory, when the kernel works on a channel slice of them (one group of a
    // grouped convolution: C, K are the group's, Cs, Ks the tensors'); 0 = the same as C / K
    int Cs = 0, Ks = 0;
    // implicit-GEMM kernel only: kernel taps that share one 64-deep reduction step (2 for at most 32 input channels, 4 for
    // at most 16; the weights are packed to match, igemm_tap_pack); 0 or 1 = a step is one tap x 64 channels
    int tap_pack = 0;
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

// Out-of-line copy of the generic tail: keeps the kernels that carry it small (it is the slow path anyway).
__device__ __noinline__ void epilogue_store8_generic(void* __restrict__ out, const Epilogue* ep, int n, int ch0, int pix,
                                                     int K, int OHW, int a0, int a1, int a2, int a3, int a4, int a5,
                                                     int a6, int a7) {
    const int a8[8] = {a0, a1, a2, a3, a4, a5, a6, a7};
    float si[8], bi[8], so[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        si[e] = ep->scale_in[ch0 + e];
        bi[e] = ep->bias ? ep->bias[ch0 + e] : 0.f;
        so[e] = ep->scale_out ? ep->scale_out[ch0 + e] : 1.f;
    }
    epilogue_store8(out, *ep, n, ch0, pix, K, OHW, a8, si, bi, so);
}

// Per-lane epilogue constants of 8 consecutive channels for the fast paths. `bias` always points at an array
// (filled with -0.0f when the layer has no bias: fma(a, s, -0.0f) == a * s bit for bit, sign of zero included).
struct Epi8 {
    float si[8], bi[8], so[8];
    unsigned qh[4];  // upper clamp of the rounded result per channel, as packed int16 pairs (epi8_clamp_init)
};

__device__ __forceinline__ void epi8_clamp_init(const Epilogue& ep, Epi8& p);

template <int EPI>
__device__ __forceinline__ void epi8_load(Epi8& p, const Epilogue& ep, int ch0) {
    const ohip_v4i* s = reinterpret_cast<const ohip_v4i*>(ep.scale_in + ch0);
    const ohip_v4i* b = reinterpret_cast<const ohip_v4i*>(ep.bias + ch0);
    ohip_v4i s0 = s[0], s1 = s[1], b0 = b[0], b1 = b[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        p.si[e] = __int_as_float(s0[e]);
        p.si[4 + e] = __int_as_float(s1[e]);
        p.bi[e] = __int_as_float(b0[e]);
        p.bi[4 + e] = __int_as_float(b1[e]);
    }
    if constexpr (EPI == EPI_I8_P8 || EPI == EPI_I8_P8_NONNEG) {
        const ohip_v4i* o = reinterpret_cast<const ohip_v4i*>(ep.scale_out + ch0);
        ohip_v4i o0 = o[0], o1 = o[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            p.so[e] = __int_as_float(o0[e]);
            p.so[4 + e] = __int_as_float(o1[e]);
        }
        if constexpr (EPI == EPI_I8_P8_NONNEG) epi8_clamp_init(ep, p);
    }
}

// requantize 8 channels and store one Byte8 element.
// NONNEG (ReLU / clip [0, hi], output scales > 0): the clamp is applied AFTER scaling and rounding, on the packed
// int16 values, instead of on the float before them. x -> trunc(fl(fl(x * so) + half)) is monotone for so > 0, so
// clamping its argument to [0, hi] equals clamping its result to [trunc(0 + half), trunc(fl(fl(hi * so) + half))]
// = [0, qh], bit for bit; qh (capped at the int8 saturation bound 127) is computed once per channel octet by
// epi8_clamp_init. Without an activation (!NONNEG) there is nothing to clamp but the int8 range.
typedef short ohip_v2s __attribute__((ext_vector_type(2)));

// the clamp of one channel pair, as epi8_clamp_init packs it (for kernels that keep the clamps of a row block in LDS)
__device__ __forceinline__ unsigned epi8_clamp_pair(const Epilogue& ep, float so0, float so1) {
    const int q0 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, so0), ep.round_half), 127);
    const int q1 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, so1), ep.round_half), 127);
    return (unsigned)(q0 & 0xffff) | ((unsigned)q1 << 16);
}

__device__ __forceinline__ void epi8_clamp_init(const Epilogue& ep, Epi8& p) {
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        const int q0 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, p.so[2 * h]), ep.round_half), 127);
        const int q1 = min((int)__fadd_rn(__fmul_rn(ep.act_hi, p.so[2 * h + 1]), ep.round_half), 127);
        p.qh[h] = (unsigned)(q0 & 0xffff) | ((unsigned)q1 << 16);
    }
}

// float -> uint32 toward zero, everything below zero (and NaN) to 0, everything above to 2^32 - 1: v_cvt_u32_f32. (As an
// instruction, not as a C++ conversion: that one is undefined for negative values.)
__device__ __forceinline__ unsigned cvt_u32_floor0(float v) {
    unsigned r;
    asm("v_cvt_u32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// LRELU: 0 = no LeakyReLU, 1 = LeakyReLU, -1 = decided by ep.lrelu at run time (a select per value)
template <bool NONNEG, int LRELU = -1>
__device__ __forceinline__ ohip_v2i epi8_quant_i8p8(const Epilogue& ep, const Epi8& p, const int (&a8)[8]) {
    int q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float v = __fmaf_rn((float)a8[e], p.si[e], p.bi[e]);
        if constexpr (!NONNEG && LRELU != 0) {
            if (LRELU == 1 || ep.lrelu) v = fmaxf(v, __fmul_rn(v, ep.act_p0));  // wave-uniform
        }
        v = __fmul_rn(v, p.so[e]);
        float adj = NONNEG ? __fadd_rn(v, ep.round_half) : __fadd_rn(v, __builtin_copysignf(ep.round_half, v));
        // toward zero, saturating. NONNEG: to UNSIGNED, which sends everything below zero to zero: the lower clamp of
        // the activation comes with the conversion, and only the upper one is left for the packed values
        if constexpr (NONNEG) q[e] = (int)cvt_u32_floor0(adj);
        else q[e] = (int)adj;
    }
    ohip_v2i pk;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        // two int32 -> two saturated int16 in one dword, clamp both halves at once, then gather the low bytes
        if constexpr (NONNEG) {
            typedef unsigned short ohip_v2us __attribute__((ext_vector_type(2)));
            ohip_v2us lo = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)q[4 * h], (unsigned)q[4 * h + 1]));
            ohip_v2us hi = __builtin_bit_cast(ohip_v2us, __builtin_amdgcn_cvt_pk_u16((unsigned)q[4 * h + 2], (unsigned)q[4 * h + 3]));
            lo = __builtin_elementwise_min(lo, __builtin_bit_cast(ohip_v2us, p.qh[2 * h]));
            hi = __builtin_elementwise_min(hi, __builtin_bit_cast(ohip_v2us, p.qh[2 * h + 1]));
            pk[h] = (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
            continue;
        }
        ohip_v2s lo = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[4 * h], q[4 * h + 1]));
        ohip_v2s hi = __builtin_bit_cast(ohip_v2s, __builtin_amdgcn_cvt_pk_i16(q[4 * h + 2], q[4 * h + 3]));
        if (NONNEG) {
            const ohip_v2s zero = {0, 0};
            lo = __builtin_elementwise_max(__builtin_elementwise_min(lo, __builtin_bit_cast(ohip_v2s, p.qh[2 * h])), zero);
            hi = __builtin_elementwise_max(__builtin_elementwise_min(hi, __builtin_bit_cast(ohip_v2s, p.qh[2 * h + 1])), zero);
        } else {
            const ohip_v2s top = {127, 127}, bot = {-127, -127};
            lo = __builtin_elementwise_max(__builtin_elementwise_min(lo, top), bot);
            hi = __builtin_elementwise_max(__builtin_elementwise_min(hi, top), bot);
        }
        pk[h] = (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x06040200u);
    }
    return pk;
}

template <bool NONNEG>
__device__ __forceinline__ void epi8_store_i8p8(int8_t* __restrict__ out, const Epilogue& ep, const Epi8& p, size_t elem,
                                                const int (&a8)[8]) {
    *reinterpret_cast<ohip_v2i*>(out + elem) = epi8_quant_i8p8<NONNEG>(ep, p, a8);
}

// dequantize 4 channels with the clamp activation (LRELU false) or LeakyReLU (true): the bits of one Float4 element
template <bool LRELU>
__device__ __forceinline__ ohip_v4i epi4_dequant_f32p4(const Epilogue& ep, const float* si, const float* bi, int a0, int a1,
                                                       int a2, int a3) {
    const int a[4] = {a0, a1, a2, a3};
    ohip_v4i r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = __fmaf_rn((float)a[e], si[e], bi[e]);
        if constexpr (LRELU) v = fmaxf(v, __fmul_rn(v, ep.act_p0));
        else v = fminf(fmaxf(v, ep.act_lo), ep.act_hi);
        r[e] = __float_as_int(v);
    }
    return r;
}

// dequantize (+clamp activation) 4 channels and store one Float4 element. FUSED: first add the residual blob's element
// if the epilogue carries one, and return the four bytes of the blob's int8 twin (float2int8(v * twin_scale)) if it
// carries one
// LRELU: 0 = clamp activation only, 1 = LeakyReLU, -1 = decided by ep.lrelu at run time (a select per value)
template <bool FUSED = false, int LRELU = -1>
__device__ __forceinline__ unsigned epi4_store_f32p4(float* __restrict__ out, const Epilogue& ep, const float* si,
                                                     const float* bi, size_t elem, int a0, int a1, int a2, int a3) {
    const int a[4] = {a0, a1, a2, a3};
    ohip_v4i r;
    unsigned q = 0;
    ohip_v4i res = {0, 0, 0, 0};
    if constexpr (FUSED)
        if (ep.residual != nullptr) res = *reinterpret_cast<const ohip_v4i*>(ep.residual + elem);  // wave-uniform
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = __fmaf_rn((float)a[e], si[e], bi[e]);
        if constexpr (LRELU != 1) v = fminf(fmaxf(v, ep.act_lo), ep.act_hi);  // (open for LeakyReLU)
        if constexpr (LRELU != 0) {
            if (LRELU == 1 || ep.lrelu) v = fmaxf(v, __fmul_rn(v, ep.act_p0));  // wave-uniform
        }
        if constexpr (FUSED) {
            if (ep.residual != nullptr) v = __fadd_rn(v, __int_as_float(res[e]));
            if (ep.twin != nullptr) {  // wave-uniform
                const float t = __fmul_rn(v, ep.twin_scale);
                const int k = (int)__fadd_rn(t, __builtin_copysignf(ep.twin_half, t));
                q |= (unsigned)(min(max(k, -127), 127) & 0xff) << (8 * e);
            }
        }
        r[e] = __float_as_int(v);
    }
    *reinterpret_cast<ohip_v4i*>(out + elem) = r;
    return q;
}

}  // namespace ohip
