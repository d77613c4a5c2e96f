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


// ---------------------------------------------------------------------------------------------------
// two elements per instruction: the same symbols from packed fp16 arithmetic
// ---------------------------------------------------------------------------------------------------
// rint(RN16(x / scale)) - min for two fp16 values at once, six packed fp16 instructions instead of some twenty
// scalar ones.  With P the power of two that brings the scale into [1, 2), S = scale * P (exact), r = RN16(1 / S)
// and X = x * P:
//   q0 = RN16(X * r)     rem = fma(-q0, S, X)     q = fma(rem, r, q0)          (all fp16, one rounding each)
//   t  = RN16(q + 1536)                   fp16 numbers in [1024, 2048) are the integers: the sum rounds q to the
//                                         nearest integer, ties to even, exactly as round() does
//   u  = t + (-512 - min)                 = 1024 + symbol, exact; the symbol is the low byte of the fp16 pattern
// q need not equal RN16(x / scale) (it does not for quotients far below 1), but rint(q) equals rint(RN16(x / scale))
// for every fp16 x and every positive fp16 scale with |x / scale| <= 512: tests/division_check_f16.c walks all of
// them on the CPU with exact fp16 arithmetic.  Without the scaling by P the remainder x - q0 * scale would need
// bits below fp16's smallest subnormal whenever x is small.  Symbols outside 0 .. 255 and minima outside int8 (the
// range the reference leaves undefined) come out as some byte, the same in every pass.
typedef _Float16 kvc_half2 __attribute__((ext_vector_type(2)));

struct KvcPackedParams {
    uint32_t P2, S2, r2, c2;       // two fp16 each: power of two, scaled scale, its reciprocal, -512 - min
};

__device__ __forceinline__ uint32_t kvc_half_bits(float v) { return (uint32_t)__half_as_ushort(__float2half_rn(v)); }

// the four fp16 constants of one group
__device__ __forceinline__ void kvc_packed_params_one(const KvcGroupParams &g, uint32_t &P, uint32_t &S, uint32_t &r, uint32_t &c)
{
    int e;
    (void)frexpf(g.scale, &e);                         // scale = f * 2^e, f in [0.5, 1)
    int a = 1 - e;
    a = a > 15 ? 15 : a;                               // 2^a itself must be an fp16 (subnormal scales stay below 1)
    const float Pf = ldexpf(1.f, a), Sf = g.scale * Pf;
    P = kvc_half_bits(Pf);
    S = kvc_half_bits(Sf);
    r = kvc_half_bits(__fdiv_rn(1.0f, Sf));
    c = kvc_half_bits(-512.f - g.min_i);
}

__device__ __forceinline__ KvcPackedParams kvc_packed_params(const KvcGroupParams &g0, const KvcGroupParams &g1)
{
    uint32_t P0, S0, r0, c0, P1, S1, r1, c1;
    kvc_packed_params_one(g0, P0, S0, r0, c0);
    kvc_packed_params_one(g1, P1, S1, r1, c1);
    KvcPackedParams p;
    p.P2 = P0 | (P1 << 16);
    p.S2 = S0 | (S1 << 16);
    p.r2 = r0 | (r1 << 16);
    p.c2 = c0 | (c1 << 16);
    return p;
}

// {x.lo, x.hi} -> {0x6400 + symbol of x.lo, 0x6400 + symbol of x.hi}
__device__ __forceinline__ uint32_t kvc_quant_pair_biased(uint32_t x, const KvcPackedParams &p)
{
#pragma clang fp contract(off)
    const kvc_half2 S = __builtin_bit_cast(kvc_half2, p.S2), r = __builtin_bit_cast(kvc_half2, p.r2);
    const kvc_half2 X = __builtin_bit_cast(kvc_half2, x) * __builtin_bit_cast(kvc_half2, p.P2);
    const kvc_half2 q0 = X * r;
    const kvc_half2 rem = __builtin_elementwise_fma(-q0, S, X);
    const kvc_half2 q = __builtin_elementwise_fma(rem, r, q0);
    const kvc_half2 magic = {(_Float16)1536.f, (_Float16)1536.f};
    const kvc_half2 t = q + magic;
    const kvc_half2 u = t + __builtin_bit_cast(kvc_half2, p.c2);
    return __builtin_bit_cast(uint32_t, u);
}

// low bytes of the two halves of a and of b: {a.b0, a.b2, b.b0, b.b2}
__device__ __forceinline__ uint32_t kvc_low_bytes4(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x06040200u); }

__device__ __forceinline__ float kvc_half_lo(uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu))); }
__device__ __forceinline__ float kvc_half_hi(uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); }
