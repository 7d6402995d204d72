/* TEST INFRASTRUCTURE -- CPU restatement of the reference's int8 convolution path.
 *
 * This file is the checker the GPU library is compared with. It is never linked into, loaded by, or used
 * as a fallback for the shipped library; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg load it.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   otter_oracle_float2int8, _quantize, _dequantize, _requantize, _conv_int32, _conv_layer_forward
 *       -> compared with the compiled reference (oracle/_ref, built from /root/reference by oracle/Makefile)
 *          where that library exists, and with golden vectors it produced (tests/golden/) everywhere else,
 *          including adversarial near-tie values; _conv_int32 additionally against an independent numpy
 *          int64 einsum (exact integer arithmetic, order independent).
 *   otter_oracle_activation types 4 (sigmoid) and 5 (mish): the reference evaluates them with polynomial
 *          exp / log (Tensor/QuantizeX86.hpp:38-58) and, built with -Ofast, an approximate-reciprocal instruction
 *          plus one Newton step for the division, so its own value depends on the CPU model; libm is used here.
 *          Pinned to that bound: against vectors written by the compiled reference
 *          (tests/test_activation_golden.py), int8 results equal but for at most one step at rounding ties
 *          (fewer than 0.2 % of the values), fp32 results within a relative 1e-5.
 *   x86 overflow artefact: for |v| >= 2^31 (or NaN) cvttps2dq returns INT_MIN, so the reference yields -127
 *          for a huge *positive* value. Restated here for completeness; callers keep to |v| < 2^31.
 *
 * Compile with -ffp-contract=off: the single-rounding multiply-adds of the reference build (GCC contracts
 * `bias + acc*scale` to vfmadd under its default -ffp-contract=fast with -mfma) are written as fmaf().
 */
#include "otter_int8_oracle.h"

#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

void otter_oracle_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int otter_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* cvttps2dq / cvttss2si: truncate toward zero; out of range or NaN -> "integer indefinite" INT_MIN */
static int32_t x86_cvtt(float v) {
    if (!(v >= -2147483648.0f && v < 2147483648.0f)) return INT_MIN;
    return (int32_t)v;
}

/* Tensor/VecIntrinsic.hpp:71-95 (float2int8_sse) and Tensor/QuantizeX86.cpp:18-23 (float2int8) */
int8_t otter_oracle_float2int8(float v, int round_mode) {
    int32_t i;
    if (round_mode == OTTER_ORACLE_ROUND_SSE) {
        float adj = v + copysignf(0.5f, v); /* one fp32 rounding, as _mm_add_ps */
        i = x86_cvtt(adj);
        /* _mm_packs_epi32 saturates to int16, then min 127 / max -127 */
    } else {
        /* (int)round(v): round half away from zero, exact */
        i = x86_cvtt(roundf(v));
    }
    if (i > 127) return 127;
    if (i < -127) return -127;
    return (int8_t)i;
}

/* Tensor/QuantizeX86.hpp:72-106 (activation_sse) / Tensor/QuantizeX86.cpp:25-45 (activation_ss) */
float otter_oracle_activation(float v, int act_type, const float* act_params) {
    switch (act_type) {
    case 1:
        return v > 0.f ? v : 0.f;
    case 2: {
        float slope = act_params ? act_params[0] : 0.1f; /* default: Tensor/ActivationLayer.hpp:56 */
        return v > 0.f ? v : v * slope;
    }
    case 3: {
        /* hard-wired 0..6, the parameters are ignored: Tensor/QuantizeX86.hpp:88-93 */
        if (v < 0.f) v = 0.f;
        if (v > 6.f) v = 6.f;
        return v;
    }
    case 4:
        return 1.f / (1.f + expf(-v));
    case 5:
        return v * tanhf(logf(expf(v) + 1.f));
    default:
        return v;
    }
}

/* Tensor/QuantizeX86.cpp:47-58,402 (packed, C%8==0 -> Byte8, SIMD rounding), :492-545 (elempack 4 -> 1,
 * scalar), :617-641 (unpacked, scalar); the layout a layer sees is decided by Tensor/Net.cpp:388-405. */
int otter_oracle_quantize_round_mode(int channels, int use_packing) {
    if (use_packing && channels % 8 == 0) return OTTER_ORACLE_ROUND_SSE;
    return OTTER_ORACLE_ROUND_EXACT;
}

/* Tensor/QuantizeX86.cpp:1177-1179 (Int8-packed depthwise result repacked to 4), :1723-1870 (elempack-4
 * source: SIMD rounding for both Byte8 and Byte outputs), :2075-2120 (elempack-1 source: scalar). The conv
 * result is elempack 4 when K%4==0 (Tensor/ConvolutionLayer.cpp:777-787), elempack 8 for depthwise pack8. */
int otter_oracle_requantize_round_mode(int in_channels, int out_channels, int groups, int use_packing) {
    if (!use_packing) return OTTER_ORACLE_ROUND_EXACT;
    if (in_channels == groups && groups == out_channels && in_channels % 8 == 0) return OTTER_ORACLE_ROUND_SSE;
    if (out_channels % 4 == 0) return OTTER_ORACLE_ROUND_SSE;
    return OTTER_ORACLE_ROUND_EXACT;
}

/* Tensor/ConvolutionLayer.cpp:667-679 */
void otter_oracle_scale_in(const float* weight_scales, int out_channels, float in_scale, float* scale_in) {
    for (int p = 0; p < out_channels; ++p) {
        if (weight_scales[p] == 0.f)
            scale_in[p] = 0.f;
        else
            scale_in[p] = 1.f / (in_scale * weight_scales[p]);
    }
}

/* Tensor/QuantizeX86.cpp:407-548: q = float2int8(x * scale[c or 0]) */
void otter_oracle_quantize(const float* x, int n, int c, int h, int w, const float* scales, int n_scales,
                           int round_mode, int8_t* out) {
    const size_t hw = (size_t)h * w;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < n; ++b)
        for (int q = 0; q < c; ++q) {
            const float s = n_scales == 1 ? scales[0] : scales[q];
            const float* p = x + ((size_t)b * c + q) * hw;
            int8_t* o = out + ((size_t)b * c + q) * hw;
            for (size_t i = 0; i < hw; ++i) o[i] = otter_oracle_float2int8(p[i] * s, round_mode);
        }
}

/* Tensor/ConvolutionUtils.hpp:173-191 */
int otter_oracle_conv_out_size(int in, int kernel, int stride, int pad, int dilation) {
    return (in + 2 * pad - dilation * (kernel - 1) - 1) / stride + 1;
}

/* The arithmetic of every int8 conv backend, stated as the reference's own scalar kernel states it
 * (Tensor/ConvolutionMM2D.cpp:553-649: zero padding, int32 accumulation of int8*int8 over c,u,v);
 * groups follow Tensor/Convolution.cpp:396-408; depthwise = Tensor/DepthwiseConvKernelInt8X86Pack.cpp:19-119. */
int otter_oracle_conv_int32(const int8_t* x, int n, int c, int h, int w, const int8_t* wt, int k, int kh, int kw,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, int groups,
                            int32_t* out) {
    if (groups < 1 || c % groups || k % groups) return -1;
    const int oh = otter_oracle_conv_out_size(h, kh, stride_h, pad_h, dil_h);
    const int ow = otter_oracle_conv_out_size(w, kw, stride_w, pad_w, dil_w);
    if (oh < 1 || ow < 1) return -1;
    const int cg = c / groups, kg = k / groups;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < n; ++b)
        for (int p = 0; p < k; ++p) {
            const int g = p / kg;
            int32_t* o = out + ((size_t)b * k + p) * oh * ow;
            for (int oy = 0; oy < oh; ++oy)
                for (int ox = 0; ox < ow; ++ox) {
                    int32_t sum = 0;
                    for (int q = 0; q < cg; ++q) {
                        const int8_t* xp = x + ((size_t)b * c + (size_t)g * cg + q) * h * w;
                        const int8_t* wp = wt + (((size_t)p * cg + q) * kh) * kw;
                        for (int u = 0; u < kh; ++u) {
                            const int iy = oy * stride_h - pad_h + u * dil_h;
                            if (iy < 0 || iy >= h) continue;
                            for (int v = 0; v < kw; ++v) {
                                const int ix = ox * stride_w - pad_w + v * dil_w;
                                if (ix < 0 || ix >= w) continue;
                                sum += (int32_t)xp[(size_t)iy * w + ix] * (int32_t)wp[u * kw + v];
                            }
                        }
                    }
                    o[(size_t)oy * ow + ox] = sum;
                }
        }
    return 0;
}

/* Tensor/QuantizeX86.cpp:851-903 (packed) / :1090-1158 (unpacked): y = acc*scale (+ bias, fused) */
void otter_oracle_dequantize(const int32_t* acc, int n, int c, int hw, const float* scale, int n_scale,
                             const float* bias, int n_bias, float* out) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < n; ++b)
        for (int q = 0; q < c; ++q) {
            const float s = n_scale == 1 ? scale[0] : scale[q];
            const int32_t* a = acc + ((size_t)b * c + q) * hw;
            float* o = out + ((size_t)b * c + q) * hw;
            if (!bias || n_bias == 0) {
                for (int i = 0; i < hw; ++i) o[i] = (float)a[i] * s;
            } else {
                const float bi = n_bias == 1 ? bias[0] : bias[q];
                for (int i = 0; i < hw; ++i) o[i] = fmaf((float)a[i], s, bi);
            }
        }
}

/* Tensor/QuantizeX86.cpp:1723-1870 (packed) / :2075-2120 (unpacked):
 * v = acc*scale_in (+bias, fused); v = act(v); q = float2int8(v*scale_out) */
void otter_oracle_requantize(const int32_t* acc, int n, int c, int hw, const float* scale_in, int n_scale_in,
                             const float* scale_out, int n_scale_out, const float* bias, int n_bias, int act_type,
                             const float* act_params, int round_mode, int8_t* out) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < n; ++b)
        for (int q = 0; q < c; ++q) {
            const float si = n_scale_in == 1 ? scale_in[0] : scale_in[q];
            const float so = n_scale_out == 1 ? scale_out[0] : scale_out[q];
            const int has_bias = bias && n_bias > 0;
            const float bi = has_bias ? (n_bias == 1 ? bias[0] : bias[q]) : 0.f;
            const int32_t* a = acc + ((size_t)b * c + q) * hw;
            int8_t* o = out + ((size_t)b * c + q) * hw;
            for (int i = 0; i < hw; ++i) {
                float v = has_bias ? fmaf((float)a[i], si, bi) : (float)a[i] * si;
                v = otter_oracle_activation(v, act_type, act_params);
                v = v * so;
                o[i] = otter_oracle_float2int8(v, round_mode);
            }
        }
}

/* the separate activation layer that follows dequantize on the fp32-output path
 * (Tensor/ConvolutionLayer.cpp:838-843; Tensor/ReluLayer.cpp, LReluLayer.cpp:45-, Relu6Layer.cpp:29-100) */
void otter_oracle_activation_f32(float* x, size_t count, int act_type, const float* act_params) {
    if (act_type == 0) return;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i) x[i] = otter_oracle_activation(x[i], act_type, act_params);
}

/* Tensor/ConvolutionLayer.cpp:754-847 */
int otter_oracle_conv_layer_forward(const void* x, int in_is_int8, int n, int c, int h, int w, const int8_t* wt,
                                    int k, int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w,
                                    int dil_h, int dil_w, int groups, const float* bias,
                                    const float* weight_scales, int n_wscales, float in_scale, float top_scale,
                                    int int8_out, int act_type, const float* act_params, int use_packing,
                                    int32_t* acc_out, void* out) {
    const int oh = otter_oracle_conv_out_size(h, kh, stride_h, pad_h, dil_h);
    const int ow = otter_oracle_conv_out_size(w, kw, stride_w, pad_w, dil_w);
    if (oh < 1 || ow < 1 || groups < 1 || c % groups || k % groups) return -1;
    const size_t in_count = (size_t)n * c * h * w, out_count = (size_t)n * k * oh * ow;

    float* ws = (float*)malloc(sizeof(float) * (size_t)k);
    float* scale_in = (float*)malloc(sizeof(float) * (size_t)k);
    for (int i = 0; i < k; ++i) ws[i] = n_wscales == 1 ? weight_scales[0] : weight_scales[i];
    otter_oracle_scale_in(ws, k, in_scale, scale_in);

    /* (1) quantize unless the blob is already int8 (:770-775) */
    const int8_t* xq = (const int8_t*)x;
    int8_t* xq_own = NULL;
    if (!in_is_int8) {
        xq_own = (int8_t*)malloc(in_count);
        otter_oracle_quantize((const float*)x, n, c, h, w, &in_scale, 1,
                              otter_oracle_quantize_round_mode(c, use_packing), xq_own);
        xq = xq_own;
    }
    /* (3) int32 accumulators */
    int32_t* acc = acc_out ? acc_out : (int32_t*)malloc(sizeof(int32_t) * out_count);
    int rc = otter_oracle_conv_int32(xq, n, c, h, w, wt, k, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w,
                                     groups, acc);
    /* (4) epilogue (:834-843) */
    if (rc == 0) {
        const int n_bias = bias ? k : 0;
        if (int8_out) {
            otter_oracle_requantize(acc, n, k, oh * ow, scale_in, k, &top_scale, 1, bias, n_bias, act_type,
                                    act_params, otter_oracle_requantize_round_mode(c, k, groups, use_packing),
                                    (int8_t*)out);
        } else {
            otter_oracle_dequantize(acc, n, k, oh * ow, scale_in, k, bias, n_bias, (float*)out);
            otter_oracle_activation_f32((float*)out, out_count, act_type, act_params);
        }
    }
    if (!acc_out) free(acc);
    free(xq_own);
    free(ws);
    free(scale_in);
    return rc;
}

/* Tensor/TensorPacking.cpp:1397-1552: [N,C,H,W] -> [N,C/p,H,W,p] */
void otter_oracle_pack(const void* src, size_t elem_bytes, int n, int c, int hw, int p, void* dst) {
    const char* s = (const char*)src;
    char* d = (char*)dst;
    const int cp = c / p;
    for (int b = 0; b < n; ++b)
        for (int q = 0; q < cp; ++q)
            for (int i = 0; i < hw; ++i)
                for (int j = 0; j < p; ++j)
                    memcpy(d + ((((size_t)b * cp + q) * hw + i) * p + j) * elem_bytes,
                           s + (((size_t)b * c + (size_t)q * p + j) * hw + i) * elem_bytes, elem_bytes);
}

void otter_oracle_unpack(const void* src, size_t elem_bytes, int n, int c, int hw, int p, void* dst) {
    const char* s = (const char*)src;
    char* d = (char*)dst;
    const int cp = c / p;
    for (int b = 0; b < n; ++b)
        for (int q = 0; q < cp; ++q)
            for (int i = 0; i < hw; ++i)
                for (int j = 0; j < p; ++j)
                    memcpy(d + (((size_t)b * c + (size_t)q * p + j) * hw + i) * elem_bytes,
                           s + ((((size_t)b * cp + q) * hw + i) * p + j) * elem_bytes, elem_bytes);
}

/* Tensor/EltwiseLayer.cpp:48-80 (sum) */
void otter_oracle_eltwise_add(const float* a, const float* b, size_t count, float* out) {
    for (size_t i = 0; i < count; ++i) out[i] = a[i] + b[i];
}

/* no pooling layer of this kind exists in the reference registry; defined as the fp32 mean over H*W */
void otter_oracle_global_avgpool(const float* x, int n, int c, int hw, float* out) {
    for (int i = 0; i < n * c; ++i) {
        double s = 0;
        for (int j = 0; j < hw; ++j) s += x[(size_t)i * hw + j];
        out[i] = (float)(s / hw);
    }
}

/* Tensor/InnerProductLayer.cpp:176- : y = W x + b in fp32 (accumulated in double here; compared by tolerance) */
void otter_oracle_inner_product(const float* x, int n, int in_f, const float* wt, const float* bias, int out_f,
                                float* out) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < n; ++b)
        for (int o = 0; o < out_f; ++o) {
            double s = bias ? bias[o] : 0.0;
            for (int i = 0; i < in_f; ++i) s += (double)x[(size_t)b * in_f + i] * wt[(size_t)o * in_f + i];
            out[(size_t)b * out_f + o] = (float)s;
        }
}
