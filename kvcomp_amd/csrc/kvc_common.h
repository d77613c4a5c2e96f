// kvc_common.h -- shared host/device definitions of libkvcomp_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdarg.h>

#include "../../include/kvcomp_hip.h"

// ---------------------------------------------------------------------------------------------------
// geometry
// ---------------------------------------------------------------------------------------------------
constexpr int KVC_WAVE = 64;               // lanes per tile = vectors per tile (include/kernels.h:13,18)
#ifndef KVC_WAVES_PER_WG_VALUE
#define KVC_WAVES_PER_WG_VALUE 4
#endif
constexpr int KVC_WAVES_PER_WG = KVC_WAVES_PER_WG_VALUE;
constexpr int KVC_WG = KVC_WAVE * KVC_WAVES_PER_WG;
constexpr int KVC_V_TOKENS = 128;          // tokens per V vector (include/kernels.h:17)
constexpr int KVC_MAX_TILE_BYTES = 8191;   // thread_info is u16 = end_byte*8 + pad (include/kernels.h:30-32)

// Payload staging area of one wave in LDS: the tile payload plus the up-to-15 bytes that precede it
// in its first 16-byte chunk, rounded up, plus two guard words for the look-ahead of the last refill.
constexpr int KVC_STAGE_BYTES = ((KVC_MAX_TILE_BYTES + 15 + 15) / 16) * 16 + 16;   // 8224
constexpr int KVC_STAGE_WORDS = KVC_STAGE_BYTES / 4;

// ---------------------------------------------------------------------------------------------------
// decode look-up table (built on the device from the decode tree, see kvc_lut.hip)
//
//   header   {lbits, lmax, n_long, group, fused_group, fused_check, OR of the symbols' fp16 bit patterns, 0}
//   long[ ]  codes longer than lbits: {code left-aligned in 32 bits, len | sym << 8}
//   entry[ ] 1 << lbits words indexed by the next lbits stream bits: len | sym << 8, or 0 when the
//            code is longer than lbits (search long[]) or the bits match no code.
//   fentry[] for the fused kernels, indexed by the next lbits stream bits taken least-significant-bit first
//            (bit j of the index = j-th next stream bit): the symbol as an fp32 bit pattern with the code
//            length in its lowest mantissa byte (zero for any integer <= 255, so read as a float the entry
//            is the symbol to within 4e-6 relative, read as a shift count it is the length).  Indices
//            whose code is longer than lbits or that match no code hold "symbol 0, length 1".
//   group    how many symbols may be decoded from one 32-bit window: floor(32 / lmax), one of 8,4,2,1.
//   fused_group / fused_check
//            the same for the fused kernels, whose window has 30 usable bits: 8 if lmax <= 3, 4 if
//            lmax <= 7 (both guaranteed to fit); for longer codes 4 with fused_check = 1 when four symbols
//            are expected to stay well inside the window (mean code length, estimated from the code
//            lengths themselves as sum len * 2^-len, at most 5.5 bits), else 2.
// ---------------------------------------------------------------------------------------------------
constexpr int KVC_LUT_MAX_BITS = 10;
constexpr int KVC_LUT_MAX_LONG = 256;
constexpr int KVC_LUT_HEADER_WORDS = 8;
constexpr int KVC_LUT_LONG_WORDS = 2 * KVC_LUT_MAX_LONG;
constexpr int KVC_LUT_ENTRY_WORDS = 1 << KVC_LUT_MAX_BITS;
constexpr int KVC_LUT_FENTRY_OFFSET = KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS + KVC_LUT_ENTRY_WORDS;
constexpr int KVC_LUT_WORDS = KVC_LUT_FENTRY_OFFSET + KVC_LUT_ENTRY_WORDS;
constexpr int KVC_LUT_BYTES = KVC_LUT_WORDS * 4;          // 10272
constexpr int KVC_TREE_MAX_NODES = 512;                   // 2 * 256 symbols - 2, rounded up

// ---------------------------------------------------------------------------------------------------
// host helpers (kvc_host.hip)
// ---------------------------------------------------------------------------------------------------
int kvc_fail(int code, const char *fmt, ...);
// Tuning knobs settable through kvc_set_option (or, before first use, KVCOMP_<NAME> in the environment).
enum KvcOption { KVC_OPT_FUSED_ROWS = 0, KVC_OPT_FUSED_TILES_PER_WAVE = 1, KVC_OPT_FUSED_PAIR_BITS = 2, KVC_OPT_FUSED_DOUBLE_WINDOW = 3, KVC_OPT_FUSED_SKEW = 4, KVC_OPT_DECODE_PIPELINED = 5, KVC_OPT_FUSED_ROUNDED = 6, KVC_OPT_ATTENTION_TAIL_IN_MERGE = 7, KVC_OPT_FUSED_MFMA = 8, KVC_OPT_FUSED_BUILTIN_DPP = 9, KVC_OPT_FUSED_SCHEDULE = 10, KVC_OPT_ENCODE_ONE_PASS = 11, KVC_OPT_FUSED_HALF_TABLE = 12, KVC_OPT_ENCODE_LOOKBACK_POLLS = 13, KVC_OPT_FUSED_SCHEDULE_V = 14, KVC_OPT_FUSED_TILES_PER_WAVE_V = 15, KVC_OPT_COUNT };
int kvc_option(KvcOption which);
int kvc_check_hip(hipError_t e, const char *what);
// A slot of the per-device scratch ring (each slot holds KVC_WS_SLOT_BYTES); used for the LUT that the
// reference-signature entry points derive from the decode tree on every call.
constexpr size_t KVC_WS_SLOT_BYTES = 16384;
int kvc_workspace_slot(void **slot, void *stream);   // stream: the one the call launches on (a recorded call gets a slot of its own)
int kvc_quant_params(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                     float eb, int8_t *d_min_i8, void *d_scale_f16, void *stream);
int kvc_expand(int is_k, int deq, const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
               const uint8_t *d_block_infos, int64_t block_infos_bytes, const uint8_t *d_thread_infos,
               int64_t thread_infos_bytes, const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_min,
               const void *d_scale, int quant_mask, void *d_out, int64_t tokens, int64_t batch, int64_t heads,
               int64_t head_dim, float *elapsed_ms, void *stream);
int kvc_launch_build_lut(const uint8_t *d_tree, int64_t tree_bytes, int tree_format, uint32_t *d_lut,
                         int n_codebooks, int64_t tree_stride_bytes, hipStream_t stream);

#define KVC_REQUIRE(cond, ...)                     \
    do {                                           \
        if (!(cond)) return kvc_fail(-1, __VA_ARGS__); \
    } while (0)
#define KVC_HIP(call)                              \
    do {                                           \
        int rc_ = kvc_check_hip((call), #call);    \
        if (rc_) return rc_;                       \
    } while (0)

// Optional event bracket implementing the reference's "returns elapsed milliseconds" contract
// (kvcomp_cuda_extension/src/kernels.cu:1026-1048).
struct KvcTimer {
    hipEvent_t a = nullptr, b = nullptr;
    hipStream_t s;
    float *out;
    KvcTimer(float *out_, hipStream_t s_) : s(s_), out(out_) {
        if (out) {
            (void)hipEventCreate(&a);
            (void)hipEventCreate(&b);
            (void)hipEventRecord(a, s);
        }
    }
    int finish() {
        if (!out) return 0;
        hipError_t e = hipEventRecord(b, s);
        if (e == hipSuccess) e = hipEventSynchronize(b);
        if (e == hipSuccess) e = hipEventElapsedTime(out, a, b);
        (void)hipEventDestroy(a);
        (void)hipEventDestroy(b);
        return kvc_check_hip(e, "event timing");
    }
};

// ---------------------------------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------------------------------
#ifdef __HIPCC__
__device__ __forceinline__ uint32_t kvc_bswap(uint32_t v) { return __builtin_bswap32(v); }

__device__ __forceinline__ float kvc_readlane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

__device__ __forceinline__ float kvc_wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Wave-wide reductions through the VALU's data-parallel lane permutes instead of LDS round trips; every lane
// of the wave must be active.  Six steps, each one instruction whose first operand is read through the
// permute: neighbours within quads (twice), quads within a row of 16 (rotate by 4, by 8: every lane of a row
// then holds the row's result), then the last lane of a row is combined into the following row (rows 1 and 3),
// and lane 31 into rows 2 and 3; lane 63 ends up with the total, which is read back as a scalar.  Rows that a
// step does not select keep their value.  A permuted read of a register needs two idle cycles after the
// instruction that wrote it, hence the s_nop between the steps (and in front: the input may have just been
// written).
#define KVC_DPP_REDUCE(op, v)                                                          \
    asm("s_nop 1\n\t" op " %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t" \
        "s_nop 1\n\t" op " %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t" \
        "s_nop 1\n\t" op " %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"           \
        "s_nop 1\n\t" op " %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"           \
        "s_nop 1\n\t" op " %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"        \
        "s_nop 1\n\t" op " %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"        \
        "s_nop 1"                                                                          \
        : "+v"(v))

__device__ __forceinline__ float kvc_wave_sum_dpp(float v)
{
    KVC_DPP_REDUCE("v_add_f32_dpp", v);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float kvc_wave_fmax_dpp(float v)
{
    KVC_DPP_REDUCE("v_max_f32_dpp", v);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ uint32_t kvc_wave_max_dpp(uint32_t v)
{
    KVC_DPP_REDUCE("v_max_u32_dpp", v);
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The kernel's argument block read again from the kernarg segment (scalar loads that hit the scalar cache): what a
// stretch of code needs of it is then live only where it is used, not in scalar registers through everything between
// (a kernel that needs more scalars than there are registers keeps the surplus in lanes of a vector register, and every
// access to those costs a vector instruction).
template <class T>
__device__ __forceinline__ const T &kvc_kernarg_again()
{
    auto p = __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return *(const T *)p;
}

// inclusive prefix sum over the 64 lanes of a wave
__device__ __forceinline__ uint32_t kvc_wave_inclusive_scan(uint32_t v, int lane)
{
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        uint32_t t = __shfl_up(v, off, 64);
        if (lane >= off) v += t;
    }
    return v;
}
#endif
