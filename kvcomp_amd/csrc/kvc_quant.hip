// kvc_quant.hip -- error-bounded block quantizer, dequantizer, symbol histogram and the dense matvec
// baseline.
//
//   kvc_quant      <- quant (utils/compute.py:93-106, src/compute.cpp:40-58) and quant_ints
//                     (utils/compute.py:74-91), which the reference runs as ~8 separate fp16 PyTorch
//                     kernels; here: min/max by wavefront reductions, then one pass that writes symbols.
//   kvc_dequant    <- (sym + min_i) * scale (models/cache/kvcomp_encode.py:146,161)
//   kvc_histogram  <- torch::bincount in build_codebook (src/huffman.cpp:105-109), with LDS atomics
//   kvc_k_mat_vec_mul <- k_mat_vec_mul (src/kernels.cu:1192-1273)
//
// Bit-exactness of the quantizer: every reference op is an fp16 tensor op, i.e. an fp32 operation on
// the exact fp16 inputs followed by one rounding to fp16.  The device code spells out exactly that
// chain; the fp32 division is IEEE (correctly rounded) and fp16/fp32 subnormals are kept.
#include "kvc_common.h"
#include "kvc_quant_math.h"

__device__ __forceinline__ float kvc_wave_min(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float kvc_wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// order-preserving float <-> uint map for atomicMin / atomicMax
__device__ __forceinline__ uint32_t kvc_f2ord(float f)
{
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float kvc_ord2f(uint32_t o)
{
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

struct KvcQuantArgs {
    const __half *x;
    int64_t NB, BS, B, H, D;
    int mask;
    float eb;
    uint8_t *sym;
    int8_t *min_i8;
    __half *scale_f16;
    __half *min_f16;       // optional
    __half *xhat;          // optional: simulated-quantization values, same shape as x
    uint32_t *minmax;      // block modes: {ord(min), ord(max)} per group
};

// Writes the symbols and/or the simulated-quantization values of two adjacent elements.
__device__ __forceinline__ void kvc_quant_store2(const KvcQuantArgs &a, int64_t i, float v0, float v1,
                                                 const KvcGroupParams &g0, const KvcGroupParams &g1)
{
    if (a.sym) {
        uchar2 o;
        o.x = kvc_quant_one(v0, g0);
        o.y = kvc_quant_one(v1, g1);
        *reinterpret_cast<uchar2 *>(a.sym + i) = o;
    }
    if (a.xhat) *reinterpret_cast<__half2 *>(a.xhat + i) = __halves2half2(kvc_quant_error_one(v0, g0), kvc_quant_error_one(v1, g1));
}

// ... of eight adjacent elements of one group (i a multiple of 8; 8- and 16-byte stores)
template <int GSTEP>   // element k belongs to group g[k * GSTEP]: 0 = one group for all eight, 1 = a group each
__device__ __forceinline__ void kvc_quant_store8(const KvcQuantArgs &a, int64_t i, const uint4 &raw, const KvcGroupParams *g)
{
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float v[8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        v[2 * k] = __half2float(__ushort_as_half((unsigned short)(w[k] & 0xffffu)));
        v[2 * k + 1] = __half2float(__ushort_as_half((unsigned short)(w[k] >> 16)));
    }
    if (a.sym) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo |= (uint32_t)kvc_quant_one(v[k], g[k * GSTEP]) << (8 * k);
            hi |= (uint32_t)kvc_quant_one(v[4 + k], g[(4 + k) * GSTEP]) << (8 * k);
        }
        *reinterpret_cast<uint2 *>(a.sym + i) = make_uint2(lo, hi);
    }
    if (a.xhat) {
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            o[k] = (uint32_t)__half_as_ushort(kvc_quant_error_one(v[2 * k], g[2 * k * GSTEP])) |
                   ((uint32_t)__half_as_ushort(kvc_quant_error_one(v[2 * k + 1], g[(2 * k + 1) * GSTEP])) << 16);
        *reinterpret_cast<uint4 *>(a.xhat + i) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

__device__ __forceinline__ void kvc_quant_minmax8(const uint4 &raw, float &mn, float &mx)
{
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const float v0 = __half2float(__ushort_as_half((unsigned short)(w[k] & 0xffffu)));
        const float v1 = __half2float(__ushort_as_half((unsigned short)(w[k] >> 16)));
        mn = fminf(mn, fminf(v0, v1));
        mx = fmaxf(mx, fmaxf(v0, v1));
    }
}

__device__ __forceinline__ void kvc_quant_publish(const KvcQuantArgs &a, int64_t g, const KvcGroupParams &gp)
{
    if (a.scale_f16) a.scale_f16[g] = gp.scale_h;
    if (a.min_i8) a.min_i8[g] = (int8_t)(int)gp.min_i;
    if (a.min_f16) a.min_f16[g] = gp.min_h;
}

// ---- per-channel groups (mask 0x1): a thread owns two adjacent channels of one block and walks the
// BS tokens twice; no cross-lane traffic at all. ------------------------------------------------------
__global__ void __launch_bounds__(KVC_WG) kvc_quant_channel_kernel(KvcQuantArgs a)
{
    const int64_t stride = a.B * a.H * a.D;
    const int64_t pairs = stride >> 1;
    const int64_t gid = (int64_t)blockIdx.x * KVC_WG + threadIdx.x;
    if (gid >= a.NB * pairs) return;
    const int64_t nb = gid / pairs, c = (gid - nb * pairs) * 2;
    const __half *p = a.x + nb * a.BS * stride + c;
    float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
    for (int64_t t = 0; t < a.BS; t++) {
        const __half2 v = *reinterpret_cast<const __half2 *>(p + t * stride);
        const float v0 = __low2float(v), v1 = __high2float(v);
        mn0 = fminf(mn0, v0); mx0 = fmaxf(mx0, v0);
        mn1 = fminf(mn1, v1); mx1 = fmaxf(mx1, v1);
    }
    const KvcGroupParams g0 = kvc_group_params(mn0, mx0, a.eb), g1 = kvc_group_params(mn1, mx1, a.eb);
    const int64_t g = nb * stride + c;
    kvc_quant_publish(a, g, g0);
    kvc_quant_publish(a, g + 1, g1);
    if (!a.sym && !a.xhat) return;                        // parameters only
    const int64_t base = nb * a.BS * stride + c;
    for (int64_t t = 0; t < a.BS; t++) {
        const __half2 v = *reinterpret_cast<const __half2 *>(p + t * stride);
        kvc_quant_store2(a, base + t * stride, __low2float(v), __high2float(v), g0, g1);
    }
}

// The same with eight adjacent channels per thread (16-byte loads, 8-byte symbol stores) for row strides that
// are a multiple of 8 and 16-byte aligned buffers.
__global__ void __launch_bounds__(KVC_WG) kvc_quant_channel8_kernel(KvcQuantArgs a)
{
    const int64_t stride = a.B * a.H * a.D;
    const int64_t octs = stride >> 3;
    const int64_t gid = (int64_t)blockIdx.x * KVC_WG + threadIdx.x;
    if (gid >= a.NB * octs) return;
    const int64_t nb = gid / octs, c = (gid - nb * octs) * 8;
    const __half *p = a.x + nb * a.BS * stride + c;
    float mn[8], mx[8];
#pragma unroll
    for (int k = 0; k < 8; k++) { mn[k] = INFINITY; mx[k] = -INFINITY; }
#pragma unroll 4
    for (int64_t t = 0; t < a.BS; t++) {
        const uint4 raw = *reinterpret_cast<const uint4 *>(p + t * stride);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float v0 = __half2float(__ushort_as_half((unsigned short)(w[k] & 0xffffu)));
            const float v1 = __half2float(__ushort_as_half((unsigned short)(w[k] >> 16)));
            mn[2 * k] = fminf(mn[2 * k], v0); mx[2 * k] = fmaxf(mx[2 * k], v0);
            mn[2 * k + 1] = fminf(mn[2 * k + 1], v1); mx[2 * k + 1] = fmaxf(mx[2 * k + 1], v1);
        }
    }
    KvcGroupParams gp[8];
    const int64_t g = nb * stride + c;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        gp[k] = kvc_group_params(mn[k], mx[k], a.eb);
        kvc_quant_publish(a, g + k, gp[k]);
    }
    if (!a.sym && !a.xhat) return;                        // parameters only
    const int64_t base = nb * a.BS * stride + c;
#pragma unroll 2
    for (int64_t t = 0; t < a.BS; t++)
        kvc_quant_store8<1>(a, base + t * stride, *reinterpret_cast<const uint4 *>(p + t * stride), gp);
}

// The simulated-quantization values of two elements from kvc_quant_pair_biased's result: u - 1024 is the fp16 symbol the
// reference keeps un-cast (rint(x / scale) - min, exact), then its two fp16 tensor ops (utils/compute.py:130):
// (symbol + min) -- the sum of two integers, exact -- times scale, one rounding.
__device__ __forceinline__ uint32_t kvc_quant_error_pair(uint32_t u, uint32_t min2, uint32_t scale2)
{
#pragma clang fp contract(off)
    const kvc_half2 bias = {(_Float16)1024.f, (_Float16)1024.f};
    const kvc_half2 sym = __builtin_bit_cast(kvc_half2, u) - bias;
    const kvc_half2 v = (sym + __builtin_bit_cast(kvc_half2, min2)) * __builtin_bit_cast(kvc_half2, scale2);
    return __builtin_bit_cast(uint32_t, v);
}
// kvc_quant_pair_biased gives the reference's integers where every quotient x / scale of the group stays within +-512
// (kvc_quant_math.h); the group's smallest and largest quotients say whether it does (false for a zero scale too).
__device__ __forceinline__ bool kvc_packed_quantizer_applies(const KvcGroupParams &g, float mx)
{
    return fabsf(g.min_i) <= 500.f && fabsf(mx * g.rcp) <= 500.f;
}
__device__ __forceinline__ uint32_t kvc_half_pair_bits(__half lo, __half hi)
{
    return (uint32_t)__half_as_ushort(lo) | ((uint32_t)__half_as_ushort(hi) << 16);
}

// Per-channel groups over blocks of 64 tokens, symbols and / or simulated-quantization values out: a thread keeps its two channels of all
// 64 tokens in registers, so the block is read once (64 loads in flight), finds minima and maxima with packed fp16
// min / max and quantizes two channels per instruction (kvc_quant_pair_biased: the same symbols as the fp32 chain for
// every fp16 input, see kvc_quant_math.h).
__global__ void __launch_bounds__(KVC_WG) kvc_quant_channel_once_kernel(KvcQuantArgs a)
{
    const int64_t stride = a.B * a.H * a.D;
    const int64_t pairs = stride >> 1;
    const int64_t gid = (int64_t)blockIdx.x * KVC_WG + threadIdx.x;
    if (gid >= a.NB * pairs) return;
    const int64_t nb = gid / pairs, c = (gid - nb * pairs) * 2;
    const int64_t base = nb * KVC_WAVE * stride + c;
    const __half *p = a.x + base;
    uint32_t raw[KVC_WAVE];
#pragma unroll
    for (int t = 0; t < KVC_WAVE; t++) raw[t] = *reinterpret_cast<const uint32_t *>(p + t * stride);
    kvc_half2 mn = __builtin_bit_cast(kvc_half2, raw[0]), mx = mn;
#pragma unroll
    for (int t = 1; t < KVC_WAVE; t++) {
        const kvc_half2 x = __builtin_bit_cast(kvc_half2, raw[t]);
        mn = __builtin_elementwise_min(mn, x);
        mx = __builtin_elementwise_max(mx, x);
    }
    const uint32_t mnw = __builtin_bit_cast(uint32_t, mn), mxw = __builtin_bit_cast(uint32_t, mx);
    const KvcGroupParams g0 = kvc_group_params(kvc_half_lo(mnw), kvc_half_lo(mxw), a.eb);
    const KvcGroupParams g1 = kvc_group_params(kvc_half_hi(mnw), kvc_half_hi(mxw), a.eb);
    const int64_t g = nb * stride + c;
    kvc_quant_publish(a, g, g0);
    kvc_quant_publish(a, g + 1, g1);
    if (kvc_packed_quantizer_applies(g0, kvc_half_lo(mxw)) && kvc_packed_quantizer_applies(g1, kvc_half_hi(mxw))) {
        const KvcPackedParams pp = kvc_packed_params(g0, g1);
        const uint32_t min2 = kvc_half_pair_bits(g0.min_h, g1.min_h), scale2 = kvc_half_pair_bits(g0.scale_h, g1.scale_h);
#pragma unroll
        for (int t = 0; t < KVC_WAVE; t++) {
            const uint32_t u = kvc_quant_pair_biased(raw[t], pp);
            if (a.sym) *reinterpret_cast<uint16_t *>(a.sym + base + t * stride) = (uint16_t)kvc_low_bytes4(u, u);
            if (a.xhat) *reinterpret_cast<uint32_t *>(a.xhat + base + t * stride) = kvc_quant_error_pair(u, min2, scale2);
        }
    } else {                                               // quotients beyond the packed arithmetic's range, or a zero scale
#pragma unroll                                             // (fully: a run-time index would move the block out of the registers)
        for (int t = 0; t < KVC_WAVE; t++) kvc_quant_store2(a, base + t * stride, kvc_half_lo(raw[t]), kvc_half_hi(raw[t]), g0, g1);
    }
}

// ---- row groups (masks 0xE, 0xC, 0x8): a group is one contiguous run of R elements; one wave per
// group, min/max by wavefront reduction. -------------------------------------------------------------
__global__ void __launch_bounds__(KVC_WG) kvc_quant_row_kernel(KvcQuantArgs a, int64_t R, int64_t groups, int wide)
{
    const int lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + (threadIdx.x >> 6);
    if (g >= groups) return;
    const __half *p = a.x + g * R;
    float mn = INFINITY, mx = -INFINITY;
    if (wide) {                                           // R a multiple of 8, all pointers 16-byte aligned
        for (int64_t i = 8 * lane; i < R; i += 8 * KVC_WAVE) kvc_quant_minmax8(*reinterpret_cast<const uint4 *>(p + i), mn, mx);
    } else {
        for (int64_t i = 2 * lane; i < R; i += 2 * KVC_WAVE) {
            const __half2 v = *reinterpret_cast<const __half2 *>(p + i);
            const float v0 = __low2float(v), v1 = __high2float(v);
            mn = fminf(mn, fminf(v0, v1));
            mx = fmaxf(mx, fmaxf(v0, v1));
        }
    }
    mn = kvc_wave_min(mn);
    mx = kvc_wave_max(mx);
    const KvcGroupParams gp = kvc_group_params(mn, mx, a.eb);
    if (lane == 0) kvc_quant_publish(a, g, gp);
    if (!a.sym && !a.xhat) return;                        // parameters only
    if (wide) {
        for (int64_t i = 8 * lane; i < R; i += 8 * KVC_WAVE) kvc_quant_store8<0>(a, g * R + i, *reinterpret_cast<const uint4 *>(p + i), &gp);
    } else {
        for (int64_t i = 2 * lane; i < R; i += 2 * KVC_WAVE) {
            const __half2 v = *reinterpret_cast<const __half2 *>(p + i);
            kvc_quant_store2(a, g * R + i, __low2float(v), __high2float(v), gp, gp);
        }
    }
}

// Row groups of 512 to 512 NIT elements (a multiple of 8, 16-byte aligned buffers), symbols and / or simulated-quantization
// values out: the
// wave keeps the row in registers (NIT 16-byte loads per lane in flight), so it is read once, and quantizes two
// elements per instruction (kvc_quant_pair_biased, as the per-channel kernel above).
template <int NIT>
__global__ void __launch_bounds__(KVC_WG) kvc_quant_row_once_kernel(KvcQuantArgs a, int64_t R, int64_t groups)
{
    const int lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + (threadIdx.x >> 6);
    if (g >= groups) return;
    const __half *p = a.x + g * R;
    uint4 raw[NIT];
#pragma unroll
    for (int j = 0; j < NIT; j++) {
        const int64_t i = 8 * lane + 512 * j;
        if (i < R) raw[j] = *reinterpret_cast<const uint4 *>(p + i);
    }
    // R >= 512 (the launcher's condition): every lane holds the row's first chunk
    kvc_half2 mn = __builtin_bit_cast(kvc_half2, raw[0].x), mx = mn;
    {
        const uint32_t w[3] = {raw[0].y, raw[0].z, raw[0].w};
#pragma unroll
        for (int k = 0; k < 3; k++) {
            const kvc_half2 x = __builtin_bit_cast(kvc_half2, w[k]);
            mn = __builtin_elementwise_min(mn, x);
            mx = __builtin_elementwise_max(mx, x);
        }
    }
#pragma unroll
    for (int j = 1; j < NIT; j++) {
        if (8 * lane + 512 * j < R) {
            const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const kvc_half2 x = __builtin_bit_cast(kvc_half2, w[k]);
                mn = __builtin_elementwise_min(mn, x);
                mx = __builtin_elementwise_max(mx, x);
            }
        }
    }
    const uint32_t mnw = __builtin_bit_cast(uint32_t, mn), mxw = __builtin_bit_cast(uint32_t, mx);
    const float lo = kvc_wave_min(fminf(kvc_half_lo(mnw), kvc_half_hi(mnw)));
    const float hi = kvc_wave_max(fmaxf(kvc_half_lo(mxw), kvc_half_hi(mxw)));
    const KvcGroupParams gp = kvc_group_params(lo, hi, a.eb);
    if (lane == 0) kvc_quant_publish(a, g, gp);
    if (!kvc_packed_quantizer_applies(gp, hi)) {           // (wave-uniform) quotients beyond the packed arithmetic's range, or a zero scale
#pragma unroll
        for (int j = 0; j < NIT; j++) {
            const int64_t i = 8 * lane + 512 * j;
            if (i < R) kvc_quant_store8<0>(a, g * R + i, raw[j], &gp);
        }
        return;
    }
    const KvcPackedParams pp = kvc_packed_params(gp, gp);
    const uint32_t min2 = kvc_half_pair_bits(gp.min_h, gp.min_h), scale2 = kvc_half_pair_bits(gp.scale_h, gp.scale_h);
#pragma unroll
    for (int j = 0; j < NIT; j++) {
        const int64_t i = 8 * lane + 512 * j;
        if (i < R) {
            const uint32_t u0 = kvc_quant_pair_biased(raw[j].x, pp), u1 = kvc_quant_pair_biased(raw[j].y, pp);
            const uint32_t u2 = kvc_quant_pair_biased(raw[j].z, pp), u3 = kvc_quant_pair_biased(raw[j].w, pp);
            if (a.sym) *reinterpret_cast<uint2 *>(a.sym + g * R + i) = make_uint2(kvc_low_bytes4(u0, u1), kvc_low_bytes4(u2, u3));
            if (a.xhat)
                *reinterpret_cast<uint4 *>(a.xhat + g * R + i) = make_uint4(kvc_quant_error_pair(u0, min2, scale2), kvc_quant_error_pair(u1, min2, scale2),
                                                                           kvc_quant_error_pair(u2, min2, scale2), kvc_quant_error_pair(u3, min2, scale2));
        }
    }
}

// ---- block groups (masks 0xF, 0xD): rows of R contiguous elements map many-to-one onto groups;
// wave-reduce each row, then merge rows with atomics on an order-preserving integer image. -----------
__device__ __forceinline__ int64_t kvc_block_group_of_row(const KvcQuantArgs &a, int64_t row)
{
    if (a.mask == KVC_MASK_K_BLOCK) return row / a.BS;                 // row = token
    const int64_t b = row % a.B;                                       // row = (token, b)
    return (row / (a.BS * a.B)) * a.B + b;
}

__global__ void __launch_bounds__(KVC_WG) kvc_quant_block_init_kernel(uint32_t *minmax, int64_t groups)
{
    const int64_t g = (int64_t)blockIdx.x * KVC_WG + threadIdx.x;
    if (g < groups) { minmax[2 * g] = 0xffffffffu; minmax[2 * g + 1] = 0u; }
}

__global__ void __launch_bounds__(KVC_WG) kvc_quant_block_minmax_kernel(KvcQuantArgs a, int64_t R, int64_t rows)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const __half *p = a.x + row * R;
    float mn = INFINITY, mx = -INFINITY;
    for (int64_t i = 2 * lane; i < R; i += 2 * KVC_WAVE) {
        const __half2 v = *reinterpret_cast<const __half2 *>(p + i);
        const float v0 = __low2float(v), v1 = __high2float(v);
        mn = fminf(mn, fminf(v0, v1));
        mx = fmaxf(mx, fmaxf(v0, v1));
    }
    mn = kvc_wave_min(mn);
    mx = kvc_wave_max(mx);
    if (lane == 0) {
        const int64_t g = kvc_block_group_of_row(a, row);
        atomicMin(&a.minmax[2 * g], kvc_f2ord(mn));
        atomicMax(&a.minmax[2 * g + 1], kvc_f2ord(mx));
    }
}

__global__ void __launch_bounds__(KVC_WG) kvc_quant_block_apply_kernel(KvcQuantArgs a, int64_t R, int64_t rows)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t g = kvc_block_group_of_row(a, row);
    const KvcGroupParams gp = kvc_group_params(kvc_ord2f(a.minmax[2 * g]), kvc_ord2f(a.minmax[2 * g + 1]), a.eb);
    // the first row of a group also publishes the group's metadata
    const bool first = a.mask == KVC_MASK_K_BLOCK ? (row % a.BS == 0) : ((row / a.B) % a.BS == 0);
    if (first && lane == 0) kvc_quant_publish(a, g, gp);
    if (!a.sym && !a.xhat) return;                        // parameters only
    const __half *p = a.x + row * R;
    for (int64_t i = 2 * lane; i < R; i += 2 * KVC_WAVE) {
        const __half2 v = *reinterpret_cast<const __half2 *>(p + i);
        kvc_quant_store2(a, row * R + i, __low2float(v), __high2float(v), gp, gp);
    }
}

extern "C" int64_t kvc_quant_groups(int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int mask)
{
    return NB * ((mask & 1) ? 1 : BS) * ((mask & 2) ? 1 : B) * ((mask & 4) ? 1 : H) * ((mask & 8) ? 1 : D);
}

extern "C" int kvc_histogram(const uint8_t *d_sym, int64_t n, int64_t *d_counts, void *stream);

static int kvc_quant_launch(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                            float eb, uint8_t *d_sym, int8_t *d_min_i8, void *d_scale_f16, void *d_min_f16,
                            void *d_xhat_f16, int64_t *d_counts, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(NB >= 0 && BS > 0 && B > 0 && H > 0 && D > 0, "bad shape");
    KVC_REQUIRE(D % 2 == 0, "head_dim must be even");
    KVC_REQUIRE(((uintptr_t)d_x_f16 & 3) == 0 && ((uintptr_t)d_sym & 1) == 0 && ((uintptr_t)d_xhat_f16 & 3) == 0,
                "quantizer buffers are misaligned");
    KVC_REQUIRE(eb > 0.f, "error bound must be positive");
    if (NB == 0) return 0;
    KvcQuantArgs a;
    a.x = reinterpret_cast<const __half *>(d_x_f16);
    a.NB = NB; a.BS = BS; a.B = B; a.H = H; a.D = D;
    a.mask = quant_mask;
    a.eb = eb;
    a.sym = d_sym;
    a.min_i8 = d_min_i8;
    a.scale_f16 = reinterpret_cast<__half *>(d_scale_f16);
    a.min_f16 = reinterpret_cast<__half *>(d_min_f16);
    a.xhat = reinterpret_cast<__half *>(d_xhat_f16);
    a.minmax = nullptr;
    const int64_t stride = B * H * D;
    if (quant_mask == KVC_MASK_CHANNEL) {
        const bool wide = stride % 8 == 0 && ((uintptr_t)a.x & 15) == 0 && ((uintptr_t)a.sym & 7) == 0 && ((uintptr_t)a.xhat & 15) == 0;
        const bool once = BS == KVC_WAVE && (a.sym != nullptr || a.xhat != nullptr);   // the block fits a thread's registers
        const int64_t threads = NB * (once || !wide ? stride / 2 : stride / 8);
        const dim3 grid((unsigned)((threads + KVC_WG - 1) / KVC_WG));
        if (once) hipLaunchKernelGGL(kvc_quant_channel_once_kernel, grid, dim3(KVC_WG), 0, stream, a);
        else if (wide) hipLaunchKernelGGL(kvc_quant_channel8_kernel, grid, dim3(KVC_WG), 0, stream, a);
        else hipLaunchKernelGGL(kvc_quant_channel_kernel, grid, dim3(KVC_WG), 0, stream, a);
    } else if (quant_mask == KVC_MASK_V_TOKEN || quant_mask == KVC_MASK_SIM_TOKEN || quant_mask == KVC_MASK_VECTOR) {
        const int64_t R = quant_mask == KVC_MASK_V_TOKEN ? stride : quant_mask == KVC_MASK_SIM_TOKEN ? H * D : D;
        const int64_t groups = NB * BS * stride / R;
        const int wide = R % 8 == 0 && ((uintptr_t)a.x & 15) == 0 && ((uintptr_t)a.sym & 7) == 0 && ((uintptr_t)a.xhat & 15) == 0;
        const dim3 grid((unsigned)((groups + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG));
        const bool once = wide && (a.sym != nullptr || a.xhat != nullptr) && R >= 512;  // the row fits a wave's registers
        if (once && R <= 512 * 8) hipLaunchKernelGGL(kvc_quant_row_once_kernel<8>, grid, dim3(KVC_WG), 0, stream, a, R, groups);
        else if (once && R <= 512 * 16) hipLaunchKernelGGL(kvc_quant_row_once_kernel<16>, grid, dim3(KVC_WG), 0, stream, a, R, groups);
        else if (once && R <= 512 * 24) hipLaunchKernelGGL(kvc_quant_row_once_kernel<24>, grid, dim3(KVC_WG), 0, stream, a, R, groups);
        else if (once && R <= 512 * 32) hipLaunchKernelGGL(kvc_quant_row_once_kernel<32>, grid, dim3(KVC_WG), 0, stream, a, R, groups);
        else hipLaunchKernelGGL(kvc_quant_row_kernel, grid, dim3(KVC_WG), 0, stream, a, R, groups, wide);
    } else if (quant_mask == KVC_MASK_K_BLOCK || quant_mask == KVC_MASK_SIM_BLOCK) {
        const int64_t R = quant_mask == KVC_MASK_K_BLOCK ? stride : H * D;
        const int64_t rows = NB * BS * stride / R;
        const int64_t groups = quant_mask == KVC_MASK_K_BLOCK ? NB : NB * B;
        KVC_REQUIRE(groups * 8 <= (int64_t)KVC_WS_SLOT_BYTES, "too many block-quantization groups (%lld) for one call", (long long)groups);
        void *slot;
        if (int rc = kvc_workspace_slot(&slot, (void *)stream)) return rc;
        a.minmax = reinterpret_cast<uint32_t *>(slot);
        const unsigned row_wgs = (unsigned)((rows + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG);
        hipLaunchKernelGGL(kvc_quant_block_init_kernel, dim3((unsigned)((groups + KVC_WG - 1) / KVC_WG)), dim3(KVC_WG), 0, stream, a.minmax, groups);
        hipLaunchKernelGGL(kvc_quant_block_minmax_kernel, dim3(row_wgs), dim3(KVC_WG), 0, stream, a, R, rows);
        hipLaunchKernelGGL(kvc_quant_block_apply_kernel, dim3(row_wgs), dim3(KVC_WG), 0, stream, a, R, rows);
    } else {
        return kvc_fail(-1, "unsupported quantization group mask 0x%x", quant_mask);
    }
    KVC_HIP(hipGetLastError());
    if (d_counts) return kvc_histogram(d_sym, NB * BS * stride, d_counts, stream_);
    return 0;
}

extern "C" int kvc_quant(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                         float eb, uint8_t *d_sym, int8_t *d_min_i8, void *d_scale_f16, void *d_min_f16,
                         int64_t *d_counts, void *stream)
{
    KVC_REQUIRE(d_sym != nullptr && d_min_i8 != nullptr && d_scale_f16 != nullptr, "output pointer is NULL");
    return kvc_quant_launch(d_x_f16, NB, BS, B, H, D, quant_mask, eb, d_sym, d_min_i8, d_scale_f16, d_min_f16, nullptr,
                            d_counts, stream);
}

// group parameters (min_i8, scale) without symbols: the first pass of the fused quantize + encode path
int kvc_quant_params(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                     float eb, int8_t *d_min_i8, void *d_scale_f16, void *stream)
{
    return kvc_quant_launch(d_x_f16, NB, BS, B, H, D, quant_mask, eb, nullptr, d_min_i8, d_scale_f16, nullptr, nullptr,
                            nullptr, stream);
}

extern "C" int kvc_quant_error(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                               float eb, void *d_xhat_f16, void *stream)
{
    KVC_REQUIRE(d_xhat_f16 != nullptr, "output pointer is NULL");
    return kvc_quant_launch(d_x_f16, NB, BS, B, H, D, quant_mask, eb, nullptr, nullptr, nullptr, nullptr, d_xhat_f16,
                            nullptr, stream);
}

// ---------------------------------------------------------------------------------------------------
// dequantizer
// ---------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(KVC_WG) kvc_dequant_kernel(const uint8_t *__restrict__ sym, const int8_t *__restrict__ min_i8,
                                                             const __half *__restrict__ scale, int64_t BS, int64_t B, int64_t H,
                                                             int64_t D, int mask, __half *__restrict__ out, int64_t n)
{
    const int64_t gBS = (mask & 1) ? 1 : BS, gB = (mask & 2) ? 1 : B, gH = (mask & 4) ? 1 : H, gD = (mask & 8) ? 1 : D;
    for (int64_t i = (int64_t)blockIdx.x * KVC_WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * KVC_WG) {
        int64_t r = i;
        const int64_t d = r % D; r /= D;
        const int64_t h = r % H; r /= H;
        const int64_t b = r % B; r /= B;
        const int64_t bs = r % BS;
        const int64_t nb = r / BS;
        const int64_t g = (((nb * gBS + ((mask & 1) ? 0 : bs)) * gB + ((mask & 2) ? 0 : b)) * gH + ((mask & 4) ? 0 : h)) * gD +
                          ((mask & 8) ? 0 : d);
        const int v = (int)sym[i] + (int)min_i8[g];
        out[i] = __float2half_rn((float)v * __half2float(scale[g]));
    }
}

extern "C" int kvc_dequant(const uint8_t *d_sym, const int8_t *d_min_i8, const void *d_scale_f16, int64_t NB, int64_t BS,
                           int64_t B, int64_t H, int64_t D, int quant_mask, void *d_out_f16, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(NB >= 0 && BS > 0 && B > 0 && H > 0 && D > 0, "bad shape");
    KVC_REQUIRE((quant_mask & ~0xF) == 0, "bad quantization group mask");
    const int64_t n = NB * BS * B * H * D;
    if (n == 0) return 0;
    int64_t wgs = (n + KVC_WG - 1) / KVC_WG;
    if (wgs > 65536) wgs = 65536;
    hipLaunchKernelGGL(kvc_dequant_kernel, dim3((unsigned)wgs), dim3(KVC_WG), 0, stream, d_sym, d_min_i8,
                       reinterpret_cast<const __half *>(d_scale_f16), BS, B, H, D, quant_mask,
                       reinterpret_cast<__half *>(d_out_f16), n);
    return kvc_check_hip(hipGetLastError(), "kvc_dequant_kernel launch");
}

// ---------------------------------------------------------------------------------------------------
// histogram
// ---------------------------------------------------------------------------------------------------
// One counter per (bin, lane & 31): counter (bin, c) lives in LDS bank c, so the lanes of a half wave never
// collide on a bank, whatever the symbol distribution (KV symbols are heavily skewed: most lanes add to the
// same one or two bins).  Only lanes l and l + 32, and the workgroup's other waves, share a counter.
// blockIdx.y selects one of several equal chunks of `n` symbols, `chunk_stride` bytes apart, each with its own
// 256 counters.
__global__ void __launch_bounds__(KVC_WG) kvc_histogram_kernel(const uint8_t *__restrict__ sym, int64_t n,
                                                               unsigned long long *__restrict__ counts, int64_t chunk_stride)
{
    __shared__ uint32_t s_bins[256 * 32];
    const int tid = threadIdx.x, col = tid & 31;
    sym += (int64_t)blockIdx.y * chunk_stride;
    counts += (int64_t)blockIdx.y * 256;
    for (int i = tid; i < 256 * 32; i += KVC_WG) s_bins[i] = 0;
    __syncthreads();
    // bytes in front of the first 16-byte boundary, whole 16-byte groups, bytes after the last one
    int64_t head = (int64_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(sym) & 15u)) & 15u);
    if (head > n) head = n;
    const int64_t nquads = (n - head) >> 4;
    const int64_t tail = n - head - (nquads << 4);
    const uint4 *w = reinterpret_cast<const uint4 *>(sym + head);
    auto add_word = [&](uint32_t v) {
        atomicAdd(&s_bins[((v & 0xffu) << 5) | col], 1u);
        atomicAdd(&s_bins[(((v >> 8) & 0xffu) << 5) | col], 1u);
        atomicAdd(&s_bins[(((v >> 16) & 0xffu) << 5) | col], 1u);
        atomicAdd(&s_bins[((v >> 24) << 5) | col], 1u);
    };
    for (int64_t i = (int64_t)blockIdx.x * KVC_WG + tid; i < nquads; i += (int64_t)gridDim.x * KVC_WG) {
        const uint4 v = w[i];
        add_word(v.x);
        add_word(v.y);
        add_word(v.z);
        add_word(v.w);
    }
    if (blockIdx.x == 0) {
        if (tid < (int)head) atomicAdd(&s_bins[((uint32_t)sym[tid] << 5) | col], 1u);
        if (tid < (int)tail) atomicAdd(&s_bins[((uint32_t)sym[head + (nquads << 4) + tid] << 5) | col], 1u);
    }
    __syncthreads();
    uint32_t c = 0;
#pragma unroll
    for (int k = 0; k < 32; k++) c += s_bins[(tid << 5) | ((k + tid) & 31)];   // rotated: thread t starts at bank t
    if (c) atomicAdd(&counts[tid], (unsigned long long)c);
}

extern "C" int kvc_histogram(const uint8_t *d_sym, int64_t n, int64_t *d_counts, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(n >= 0, "negative length");
    if (n == 0) return 0;
    int64_t wgs = (n / 16 + KVC_WG * 8 - 1) / (KVC_WG * 8);   // ~128 symbols per thread, 2^32 per workgroup at most
    if (wgs < 1) wgs = 1;
    if (wgs > 4096) wgs = 4096;
    KVC_REQUIRE(n / wgs < (1ll << 31), "input too large for 32-bit workgroup counters");
    hipLaunchKernelGGL(kvc_histogram_kernel, dim3((unsigned)wgs), dim3(KVC_WG), 0, stream, d_sym, n,
                       reinterpret_cast<unsigned long long *>(d_counts), (int64_t)0);
    return kvc_check_hip(hipGetLastError(), "kvc_histogram_kernel launch");
}

// d_counts[c * 256 + s] += occurrences of symbol s among d_sym[c * chunk_bytes .. (c + 1) * chunk_bytes)
extern "C" int kvc_histogram_chunks(const uint8_t *d_sym, int64_t chunk_bytes, int64_t n_chunks, int64_t *d_counts, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(chunk_bytes >= 0 && n_chunks >= 0 && n_chunks <= 65535, "bad chunk geometry (%lld chunks of %lld bytes)",
                (long long)n_chunks, (long long)chunk_bytes);
    if (chunk_bytes == 0 || n_chunks == 0) return 0;
    int64_t wgs = (chunk_bytes / 16 + KVC_WG * 8 - 1) / (KVC_WG * 8);
    if (wgs < 1) wgs = 1;
    if (wgs > 4096) wgs = 4096;
    KVC_REQUIRE(chunk_bytes / wgs < (1ll << 31), "chunk too large for 32-bit workgroup counters");
    hipLaunchKernelGGL(kvc_histogram_kernel, dim3((unsigned)wgs, (unsigned)n_chunks), dim3(KVC_WG), 0, stream, d_sym,
                       chunk_bytes, reinterpret_cast<unsigned long long *>(d_counts), chunk_bytes);
    return kvc_check_hip(hipGetLastError(), "kvc_histogram_kernel launch");
}

// ---------------------------------------------------------------------------------------------------
// dense matvec baseline: out[t,b,h] = sum_i k[t,b,h,i] * q[b,h,i], fp32 accumulation.
// A row of head_dim halves is read by head_dim/8 adjacent lanes with 16-byte loads.
// ---------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(KVC_WG) kvc_k_mat_vec_mul_kernel(const __half *__restrict__ k, const __half *__restrict__ q,
                                                                   __half *__restrict__ out, int64_t rows, int bh, int D)
{
    const int lpr = D >> 3;                    // lanes per row (power of two, <= 16)
    const int rpw = KVC_WG / lpr;              // rows per workgroup pass
    const int sub = threadIdx.x % lpr;
    for (int64_t row = (int64_t)blockIdx.x * rpw + threadIdx.x / lpr; row < rows; row += (int64_t)gridDim.x * rpw) {
        const uint4 kv = *reinterpret_cast<const uint4 *>(k + row * D + sub * 8);
        const uint4 qv = *reinterpret_cast<const uint4 *>(q + (row % bh) * D + sub * 8);
        const __half2 *kh = reinterpret_cast<const __half2 *>(&kv), *qh = reinterpret_cast<const __half2 *>(&qv);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc = fmaf(__low2float(kh[j]), __low2float(qh[j]), acc);
            acc = fmaf(__high2float(kh[j]), __high2float(qh[j]), acc);
        }
        for (int off = lpr >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (sub == 0) out[row] = __float2half_rn(acc);
    }
}

extern "C" int kvc_k_mat_vec_mul(const void *d_k_f16, const void *d_q_f16, void *d_out_f16, int64_t tokens, int64_t batch,
                                 int64_t heads, int64_t head_dim, float *elapsed_ms, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128, "head_dim must be 16, 32, 64 or 128");
    KVC_REQUIRE(((uintptr_t)d_k_f16 & 15) == 0 && ((uintptr_t)d_q_f16 & 15) == 0, "k and q must be 16-byte aligned");
    const int64_t rows = tokens * batch * heads;
    if (rows == 0) {
        if (elapsed_ms) *elapsed_ms = 0.f;
        return 0;
    }
    const int rpw = KVC_WG / (int)(head_dim / 8);
    int64_t wgs = (rows + rpw - 1) / rpw;
    if (wgs > 16384) wgs = 16384;
    KvcTimer timer(elapsed_ms, stream);
    hipLaunchKernelGGL(kvc_k_mat_vec_mul_kernel, dim3((unsigned)wgs), dim3(KVC_WG), 0, stream,
                       reinterpret_cast<const __half *>(d_k_f16), reinterpret_cast<const __half *>(d_q_f16),
                       reinterpret_cast<__half *>(d_out_f16), rows, (int)(batch * heads), (int)head_dim);
    KVC_HIP(hipGetLastError());
    return timer.finish();
}

// ---------------------------------------------------------------------------------------------------
// plain device-to-device copy of a known size: the yardstick that the HBM traffic counters
// (FETCH_SIZE / WRITE_SIZE) are scaled against when a profile of this library is read.
// ---------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(KVC_WG) kvc_calibration_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t n16)
{
    for (int64_t i = (int64_t)blockIdx.x * KVC_WG + threadIdx.x; i < n16; i += (int64_t)gridDim.x * KVC_WG) dst[i] = src[i];
}

extern "C" int kvc_calibration_copy(void *d_dst, const void *d_src, int64_t bytes, void *stream_)
{
    KVC_REQUIRE(bytes >= 0 && bytes % 16 == 0, "size must be a multiple of 16");
    KVC_REQUIRE(((uintptr_t)d_dst & 15) == 0 && ((uintptr_t)d_src & 15) == 0, "pointers must be 16-byte aligned");
    if (bytes == 0) return 0;
    int64_t wgs = (bytes / 16 + KVC_WG - 1) / KVC_WG;
    if (wgs > 8192) wgs = 8192;
    hipLaunchKernelGGL(kvc_calibration_copy_kernel, dim3((unsigned)wgs), dim3(KVC_WG), 0, (hipStream_t)stream_,
                       reinterpret_cast<const uint4 *>(d_src), reinterpret_cast<uint4 *>(d_dst), bytes / 16);
    return kvc_check_hip(hipGetLastError(), "kvc_calibration_copy_kernel launch");
}
