// kvc_quant_math.h -- the scalar arithmetic of the reference quantizer (utils/compute.py:74-106), spelled out
// so that every step is the fp32 operation on exact fp16 inputs followed by one rounding to fp16 that the
// reference's fp16 tensor ops perform.  Shared by the quantizer kernels and the fused quantize + encode kernels.
#pragma once
#include "kvc_common.h"

// ---------------------------------------------------------------------------------------------------
// scalar pieces of the reference arithmetic
// ---------------------------------------------------------------------------------------------------
struct KvcGroupParams {
    float scale;     // exact value of the fp16 scale
    float min_i;     // exact value of the fp16 rounded min / scale
    float rcp;       // RN32(1 / scale), for kvc_div_by_scale
    __half scale_h, min_h;
};

// RN32(x / scale) for an fp16-valued x and an fp16-valued scale, in three instructions instead of the dozen of
// a general IEEE division: q0 = RN(x * r), the remainder x - q0 * scale is exact in one FMA, and one more FMA
// corrects q0 (Markstein's sequence; r must be the correctly rounded reciprocal).  Checked exhaustively on
// the CPU against x / scale for all 63 488 finite fp16 x and all 31 743 positive finite fp16 scales
// (2.0e9 pairs): bit-identical everywhere except that x = -0 gives +0 instead of -0, which no output of the
// quantizer can tell apart (the symbol is an integer cast, and -0 + min = +0 + min in the dequantized value).
__device__ __forceinline__ float kvc_div_by_scale(float x, const KvcGroupParams &g)
{
    const float q0 = __fmul_rn(x, g.rcp);
    const float rem = __fmaf_rn(-q0, g.scale, x);
    return __fmaf_rn(rem, g.rcp, q0);
}

__device__ __forceinline__ KvcGroupParams kvc_group_params(float mn, float mx, float eb)
{
    KvcGroupParams g;
    const __half range = __float2half_rn(mx - mn);                          // (max_ - min_)
    g.scale_h = __float2half_rn(__half2float(range) * eb);                  // * quant_scale_rel
    g.scale = __half2float(g.scale_h);
    g.rcp = __fdiv_rn(1.0f, g.scale);
    const __half mq = __float2half_rn(__fdiv_rn(mn, g.scale));              // min_ / quant_scale
    g.min_h = __float2half_rn(rintf(__half2float(mq)));                     // .round_()
    g.min_i = __half2float(g.min_h);
    return g;
}

__device__ __forceinline__ __half kvc_quant_one_f16(float x, const KvcGroupParams &g)
{
    const __half q = __float2half_rn(kvc_div_by_scale(x, g));              // tensor / quant_scale
    const __half qi = hrint(q);                                             // .round_() (half to even, exact in fp16)
    return __hsub(qi, g.min_h);                                             // quant_ints - min_ints: both integers, so
                                                                            // the fp16 difference is the rounded exact one
}

__device__ __forceinline__ uint8_t kvc_quant_one(float x, const KvcGroupParams &g)
{
    return (uint8_t)(int)__half2float(kvc_quant_one_f16(x, g));             // .to(torch.uint8)
}

// The value the simulated-quantization path keeps (utils/compute.py:130): (quant_int + min_quant) * quant_scale,
// two fp16 tensor ops on the un-cast fp16 symbol and minimum.
__device__ __forceinline__ __half kvc_quant_error_one(float x, const KvcGroupParams &g)
{
    const __half s = kvc_quant_one_f16(x, g);
    const __half sum = __float2half_rn(__half2float(s) + g.min_i);
    return __float2half_rn(__half2float(sum) * g.scale);
}

