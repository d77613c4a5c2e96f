// kvc_fused_common.h -- pieces shared by the fused decode + matvec kernels (kvc_fused.hip: fp32 FMA loops and plain
// decode; kvc_fused_mfma_impl.h: matrix-core loops): launch arguments, the one-tile-ahead fetch, payload staging.
#pragma once
#include "kvc_tile.h"

#include <mutex>
#include <type_traits>

constexpr int KVC_SCHED_SEGMENTS = 4;

struct KvcFusedArgs {
    KvcStreamArgs s;
    const int8_t *min_i8;
    const __half *scale;
    int quant_mask;
    const __half *x;     // K: q [batch, q_heads, head_dim];  V: p [batch, q_heads, tokens]
    void *out;           // K: scores [batch, q_heads, tokens]; V: partial [tokens/128, batch, q_heads, head_dim]
    int out_f32;         // 0: fp16 (reference layout), 1: fp32
    int64_t out_stride;  // K: elements between the score rows of two query heads (>= tokens)
    // softmax kinds of the V kernel: instead of p it reads raw fp32 scores and forms, per 128-token group and
    // query head, m = max(score * sm_scale), w = exp(score * sm_scale - m), l = sum w; the partial is the
    // w-weighted sum and (m, l) go to ml[group][batch][q_head][2]
    const float *scores;
    int64_t scores_stride;
    float sm_scale;
    float *ml;
    int64_t tokens;
    int batch, kv_heads, q_heads, head_dim;
    int table_words;     // LDS words reserved for the fused table (>= 1 << lbits of every codebook used)
    int pack_words;      // LDS words per wave reserved for the packed tile payload (multiple of 4)
    int pack_logical;    // payload words (lead words included) that fit there; fewer than pack_words when skewed
    int skew;            // 0, or 2: every 32 payload words are followed by a copy of the next two (see kvc_skewed)
    int row_words;       // LDS words per lane stream (odd); 0 = decode from the packed payload
    int pair_bits;       // index width of the two-symbol table the host made room for; 0 = none
    int double_window;   // refill 64 stream bits at a time where the vector length allows
    int builtin_dpp;     // fp32-FMA kernels: lane permutes through the compiler's intrinsic instead of inline assembly
    int half_table;      // matrix-core kernels: two-byte table entries for codes of 6 or 7 bits
    // kvc_expand_kernel (plain decode, decode + dequantize): no x; the operand table holds {scale, min} per element
    // Rounded mode of the matvec kernels: every (sym + min) * scale is rounded to fp16 before it meets q / p, as the
    // reference's dequantizer does (models/cache/kvcomp_encode.py:146); the operand table then holds
    // {min, scale, weight of each query head} per element and nothing is folded into a constant term.
    int rounded;
    int expand;          // 0: matvec kernels; 1: symbols out (uint8); 2: dequantized values out (fp16)
    int out_words;       // LDS words per wave for the 32-element output slab
    // Matrix-core kernels, one codebook per stream: 1-D grid over the row-major tile sequence in sched_nseg segments
    // (0: the 2-D grid of kvc_grid).  Segment k = workgroups sched_wg[k] .. sched_wg[k + 1] - 1, whose waves take
    // sched_run[k] consecutive tiles each, starting at tile sched_tile[k]; sched_tile[sched_nseg] = number of tiles.
    int sched_nseg;
    int sched_run[KVC_SCHED_SEGMENTS];
    int sched_wg[KVC_SCHED_SEGMENTS + 1];
    int sched_tile[KVC_SCHED_SEGMENTS + 1];
};

// Workgroups per CU (= waves per SIMD) each matvec kernel is compiled for.  With one query head per KV head the
// decode loops wait on LDS round trips and every further wave pays, so those kernels get the most their register
// demand allows without spilling (kinds 2 - 4 carry a second operand table or the softmax).  With four query heads
// the four FMAs per symbol hide the round trip; measured, 4 and 5 waves tie and 6 or 7 are 6 - 8 % slower.
constexpr int kvc_fused_occupancy(int rep, int kind)
{
    const bool two_slots = kind == 2 || kind == 4;
    return rep == 1 ? (kind == 1 ? 8 : 7) : (rep == 2 || (rep == 4 && !two_slots)) ? 5 : 1;
}
#ifndef KVC_FUSED_OCC
#define KVC_FUSED_OCC(REP, KIND) kvc_fused_occupancy(REP, KIND)
#endif
#ifndef KVC_MFMA_OCC_K1
#define KVC_MFMA_OCC_K1 8
#endif
#ifndef KVC_MFMA_OCC_V1
#define KVC_MFMA_OCC_V1 6
#endif
constexpr int kvc_fused_mfma_occupancy(int rep, int kind)
{
    // (four query heads, K: the kernel needs 80 registers, which leave six waves; with a bound of five the register
    // allocator settles on 81 and the sixth wave is lost: 46 -> 49 us at batch 16 x 8 KV heads x 8192 tokens)
    // (one query head, V: seven waves.  Tiles of one head each -- head_dim a multiple of 64 --: 65 registers, 37.7 -> 36.4 us
    // at batch 8 x 32 heads x 128 x 4096 tokens; eight waves fit too, with 30 spilled scalars, and measured no better.
    // Tiles that may straddle two heads, softmax on the fly: 72 registers without a spill only in a translation unit of
    // its own, kvc_fused_mfma_v96.hip; 71.7 -> 68.4 us at batch 4 x 32 heads x 96 x 32 768 tokens.)
    return rep == 1 ? (kind == 0 ? KVC_MFMA_OCC_K1 : (kind == 1 || kind == 3 || kind == 4) ? KVC_MFMA_OCC_V1 + 1 : KVC_MFMA_OCC_V1)
                    : (rep == 4 && kind == 0) ? 6 : kvc_fused_occupancy(rep, kind);
}
constexpr int KVC_PRE_CHUNKS = 4;     // 16-byte chunks per lane fetched one tile ahead (4 KiB of payload)
constexpr int KVC_PACK_LEAD = 4;      // zero words in front of the packed payload: bit positions never drop below 2

// How the (scale, minimum) pairs of a lane's two elements (2 * lane and 2 * lane + 1) lie in memory: next to each
// other (one 4-byte and one 2-byte load fetch both), the same pair for both elements, or anywhere.
enum { KVC_PAIR_SEPARATE = 0, KVC_PAIR_ADJACENT = 1, KVC_PAIR_SAME = 2 };

// What a tile needs from global memory, fetched into registers one tile ahead of its use.
template <int REP, int SLOTS, int XW>
struct KvcRaw {
    uint4 pay[KVC_PRE_CHUNKS];        // payload chunks lane, lane + 64, ...
    uint32_t off, bn;                 // block_info, clamped to the payload buffer (wave-uniform)
    uint32_t ti_cur;                  // thread_info of this lane (the previous lane's comes through a lane shift)
    // operands of elements 2 * lane and 2 * lane + 1 (K: channels, V: tokens of the 128-token group), as loaded:
    uint32_t scw[SLOTS][2];           // quantization scales (fp16 bits): see scale_bits
    uint32_t mnw[SLOTS][2];           // quantization minima (int8): see min_int
    uint32_t x[SLOTS][REP][XW];       // per query head: q / p (two fp16 in one word), or two fp32 scores
    __device__ __forceinline__ uint32_t scale_bits(int s, int half, int mode) const
    {
        if (mode == KVC_PAIR_ADJACENT) return half ? scw[s][0] >> 16 : scw[s][0] & 0xffffu;
        if (mode == KVC_PAIR_SAME) return scw[s][0] & 0xffffu;
        return scw[s][half] & 0xffffu;
    }
    __device__ __forceinline__ int min_int(int s, int half, int mode) const
    {
        if (mode == KVC_PAIR_ADJACENT) return (int)(int8_t)(mnw[s][0] >> (8 * half));
        if (mode == KVC_PAIR_SAME) return (int)(int8_t)mnw[s][0];
        return (int)(int8_t)mnw[s][half];
    }
};
// Nothing in it is touched before the tile is staged: any arithmetic on a loaded value would make the wave
// wait for the load at that point and the fetch would no longer overlap the decode of the previous tile.

// LDS traffic between the lanes of one wave needs no barrier (a wave's LDS operations complete in order);
// this only keeps the compiler from moving accesses across the hand-over.
__device__ __forceinline__ void kvc_wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// memory byte j of a word carries stream bits 8j .. 8j+7, most significant first: a byte swap followed by a
// full bit reversal leaves stream bit k of the word at bit k
__device__ __forceinline__ uint32_t kvc_stream_word(uint32_t raw) { return __brev(kvc_bswap(raw)); }

// Skewed packed payload.  Lane l starts about l mean-stream-lengths into the payload, so when a small
// multiple of that length is close to 32 words, every k-th lane reads the same bank at every refill.  With
// two spare words after every 32 (holding a copy of the two words that follow, so that the three-word read
// of a refill never has to jump), streams 32 words apart land two banks apart instead.
//   word w of the payload lives at w + skew * (w >> 5), skew = 2 (or 0: plain layout)
__device__ __forceinline__ uint32_t kvc_skewed(uint32_t w, uint32_t skew) { return __umul24(w >> 5, skew) + w; }

// Byte address in LDS of payload word u >> 5 for a refill.  No clamp: a lane's position cannot pass its start
// by more than 128 symbols x 10 bits, and the workgroup's LDS ends with that much slack (KVC_LDS_SLACK_WORDS),
// so even a corrupt stream only ever reads this workgroup's own LDS.
typedef __attribute__((address_space(3))) uint32_t kvc_lds_word;
template <bool SKEW>
__device__ __forceinline__ uint32_t kvc_refill_address(uint32_t stage_base, uint32_t u)
{
    const uint32_t a = u >> 5;
    if (SKEW) return (a << 2) + (__umul24(u >> 10, 8u) + stage_base);     // + 2 words per 32
    return (a << 2) + stage_base;
}
constexpr int KVC_LDS_SLACK_WORDS = 48;

// Rounded mode: RN16((sym + min) * scale) as the reference's dequantizer computes it (sym + min exactly, one
// rounding of the product).  Both steps are fp16 instructions: the sum of two small integers is exact in fp16
// and an fp16 multiplication rounds the exact product once.  `ms` = {min, scale} as two fp16 in one word.
__device__ __forceinline__ float kvc_rounded_value(__half sym, uint32_t ms)
{
    const __half mn = __ushort_as_half((unsigned short)(ms & 0xffffu)), sc = __ushort_as_half((unsigned short)(ms >> 16));
    return __half2float(__hmul(__hadd(sym, mn), sc));
}

template <int REP>
struct KvcVec {
    float v[REP];
};

// LDS accessed by its byte offset: the table's offset is a multiple of its size, so "window bits | offset"
// is the entry's address.
typedef __attribute__((address_space(3))) uint32_t kvc_lds_u32;
typedef __attribute__((address_space(3))) uint16_t kvc_lds_u16;

// compile-time loop: body(std::integral_constant<int, 0>) ... body(std::integral_constant<int, N - 1>)
template <int N, int I = 0, class Body>
__device__ __forceinline__ void kvc_static_for(Body &&body)
{
    if constexpr (I < N) {
        body(std::integral_constant<int, I>{});
        kvc_static_for<N, I + 1>(body);
    }
}

// -- tile geometry ------------------------------------------------------------------------------------
// KIND 0: K tile (64 tokens x head_dim channels of one (batch, head); lane = token)
// KIND 1: V tile (128 tokens x 64 flat channels; lane = channel), head_dim a multiple of 64: one head per tile
// KIND 2: V tile with any other head_dim: the 64 channels may straddle two heads (two operand tables)
// KIND 3, 4: as 1, 2 but with the softmax over the group's scores computed on the fly
template <int KIND>
struct KvcGeom {
    static constexpr bool IS_K = KIND == 0;
    static constexpr int SLOTS = (KIND == 2 || KIND == 4) ? 2 : 1;
    static constexpr bool SOFTMAX = KIND >= 3;
    static constexpr int XW = SOFTMAX ? 2 : 1;
};

template <int KIND>
__device__ __forceinline__ int kvc_pair_mode(const KvcFusedArgs &a)
{
    if (KIND == 0) return a.quant_mask == KVC_MASK_CHANNEL ? KVC_PAIR_ADJACENT : KVC_PAIR_SAME;
    if (a.quant_mask == KVC_MASK_V_TOKEN) return KVC_PAIR_ADJACENT;
    if (a.quant_mask == KVC_MASK_SIM_TOKEN) return a.batch == 1 ? KVC_PAIR_ADJACENT : KVC_PAIR_SEPARATE;
    return a.batch * a.kv_heads == 1 ? KVC_PAIR_ADJACENT : KVC_PAIR_SEPARATE;           // KVC_MASK_VECTOR
}

// Loads relative to a wave-uniform base with a 32-bit per-lane byte offset: the base stays in scalar registers and
// the address costs no 64-bit vector arithmetic.
template <class T>
__device__ __forceinline__ T kvc_load_at(const void *uniform_base, uint32_t byte_offset)
{
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(uniform_base) + byte_offset);
}

// Where a tile lies: its row and column in the tile grid and what follows from the column -- the (batch entry, head)
// it belongs to and, for a V tile, the first of its 64 channels inside that head.  Working these out from the column
// takes integer divisions, for which the hardware has no scalar instruction (each becomes some fifteen vector
// instructions, wave-uniform or not); stepping to the next tile of the row-major sequence takes a few scalar additions.
struct KvcTilePos {
    int row, col;
    int b, h;       // K: the tile's (batch entry, kv head); V: those of the tile's first channel
    int d0;         // V: the first channel's index inside head h (K: 0)
};

template <bool IS_K>
__device__ __forceinline__ KvcTilePos kvc_tile_pos(const KvcFusedArgs &a, int row, int col)
{
    KvcTilePos p;
    p.row = row;
    p.col = col;
    if (IS_K) {
        p.b = col / a.kv_heads;
        p.h = col - p.b * a.kv_heads;
        p.d0 = 0;
    } else {
        const int c0 = col * KVC_WAVE, bh = c0 / a.head_dim;
        p.d0 = c0 - bh * a.head_dim;
        p.b = bh / a.kv_heads;
        p.h = bh - p.b * a.kv_heads;
    }
    return p;
}

template <bool IS_K>
__device__ __forceinline__ KvcTilePos kvc_tile_after(const KvcFusedArgs &a, KvcTilePos p)
{
    p.col++;
    if (p.col == a.s.cols) {                                // the rows' tiles cover all (batch entry, head) pairs exactly
        p.col = 0;
        p.row++;
        p.b = p.h = p.d0 = 0;
        return p;
    }
    if (IS_K) {
        p.h++;
    } else {
        p.d0 += KVC_WAVE;
        if (p.d0 < a.head_dim) return p;
        p.d0 -= a.head_dim;
        p.h++;
        while (p.d0 >= a.head_dim) {                        // heads narrower than a tile
            p.d0 -= a.head_dim;
            p.h++;
        }
    }
    while (p.h >= a.kv_heads) {
        p.h -= a.kv_heads;
        p.b++;
    }
    return p;
}

// (batch entry, head) of a V tile's second head (the one its channels past a head boundary belong to), clamped to the
// last pair: the tile that ends a row has no second head and must not make one up.
__device__ __forceinline__ void kvc_second_head(const KvcFusedArgs &a, const KvcTilePos &p, int &b, int &h)
{
    b = p.b;
    h = p.h + 1;
    if (h == a.kv_heads) {
        if (b + 1 < a.batch) b++, h = 0;
        else h = p.h;
    }
}

// Issue the global loads of tile (row, col).  bi_off / bi_bn: the tile's block_info words.
// Parameters of a V tile's two elements per lane where every token has groups of its own per batch entry (or per batch
// entry and head): two 2-byte and two 1-byte loads.
template <class Raw>
__device__ __forceinline__ void kvc_fetch_separate_params(const KvcFusedArgs &a, int row, int b, int h, int lane, int s, Raw &raw)
{
    const int64_t tk0 = (int64_t)row * KVC_V_TOKENS;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        // group of token tk0 + t: (tk0 + t) * batch + b, times kv_heads + h for per-vector groups
        const int64_t per = a.quant_mask == KVC_MASK_SIM_TOKEN ? a.batch : (int64_t)a.batch * a.kv_heads;
        const int64_t g0 = a.quant_mask == KVC_MASK_SIM_TOKEN ? tk0 * per + b : tk0 * per + (int64_t)b * a.kv_heads + h;
        const uint32_t t = 2u * (uint32_t)lane + half;
        raw.scw[s][half] = kvc_load_at<uint16_t>(a.scale + g0, 2u * t * (uint32_t)per);
        raw.mnw[s][half] = kvc_load_at<uint8_t>(a.min_i8 + g0, t * (uint32_t)per);
    }
}

// `skip_x`: bit s set = the weights of head slot s are not needed (the wave still has that head's operand table).
// LATE_SECOND: the separate-groups parameters of a tile's second head are left to the caller, who fetches them when the
// tile is staged (kvc_fetch_separate_params): four registers less to hold through the previous tile's decode loops.
template <int REP, int KIND, int EXPAND = 0, bool LATE_SECOND = false>
__device__ __forceinline__ void kvc_fetch_tile(const KvcFusedArgs &a, const KvcTilePos &pos, uint32_t bi_off, uint32_t bi_bn,
                                               int lane, KvcRaw<REP, KvcGeom<KIND>::SLOTS, KvcGeom<KIND>::XW> &raw, int skip_x = 0)
{
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    const int row = pos.row, col = pos.col;
    const int64_t tile = (int64_t)row * a.s.cols + col;                 // wave-uniform, like everything derived from it
    const int D = a.head_dim;
    // sizes are clamped so that corrupt metadata yields wrong symbols, never an out-of-bounds access
    uint32_t off = bi_off, bn = bi_bn & 0xffffu;
    if (bn > (uint32_t)KVC_MAX_TILE_BYTES) bn = KVC_MAX_TILE_BYTES;
    if ((int64_t)off >= a.s.enc_bytes) bn = 0;
    else if ((int64_t)off + bn > a.s.enc_bytes) bn = (uint32_t)(a.s.enc_bytes - off);
    raw.off = off;
    raw.bn = bn;
    raw.ti_cur = kvc_load_at<uint16_t>(a.s.thread_infos + tile * KVC_WAVE, 2u * (uint32_t)lane);
    // payload: whole aligned 16-byte chunks that each hold at least one payload byte (such reads never leave
    // the pages the payload lives in)
    const uint8_t *src = a.s.enc + off;
    const uint32_t head = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);
    const uint32_t nchunks = bn ? (head + bn + 15u) >> 4 : 0u;
    const uint8_t *g = src - head;
#pragma unroll
    for (int j = 0; j < KVC_PRE_CHUNKS; j++) {
        const uint32_t c = (uint32_t)lane + 64u * j;
        if (c < nchunks) raw.pay[j] = kvc_load_at<uint4>(g, 16u * c);
    }
    // operands; lanes past the end of a short vector load the last pair (ignored when staged)
    const int mode = kvc_pair_mode<KIND>(a);
    if (KIND == 0) {
        const int b = pos.b, h = pos.h;
        const uint32_t e0 = (uint32_t)(2 * lane < D ? 2 * lane : D - 2);
        if (EXPAND != 1) {                                     // symbols out: no quantization parameters
            // per-channel pairs, or one pair per 64-token block (kernels.cu:771-772)
            if (mode == KVC_PAIR_ADJACENT) {
                raw.scw[0][0] = kvc_load_at<uint32_t>(a.scale + tile * D, 2u * e0);
                raw.mnw[0][0] = kvc_load_at<uint16_t>(a.min_i8 + tile * D, e0);
            } else {
                raw.scw[0][0] = kvc_load_at<uint16_t>(a.scale + row, 0u);
                raw.mnw[0][0] = kvc_load_at<uint8_t>(a.min_i8 + row, 0u);
            }
        }
        if (EXPAND == 0) {
#pragma unroll
            for (int r = 0; r < REP; r++)
                raw.x[0][r][0] = kvc_load_at<uint32_t>(a.x + ((int64_t)b * a.q_heads + h * REP + r) * D, 2u * e0);
        }
    } else {
        const int64_t tk0 = (int64_t)row * KVC_V_TOKENS;       // the group's first token; this lane's are tk0 + 2 lane (+ 1)
        const bool straddles = pos.d0 + KVC_WAVE > D;          // wave-uniform
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            if (s == 1 && !straddles) continue;                // the second head's operands are not needed
            int b = pos.b, h = pos.h;
            if (s == 1) kvc_second_head(a, pos, b, h);         // (unused by a tile that ends the row)
            if (EXPAND != 1) {
                if (mode == KVC_PAIR_ADJACENT) {               // one group per token, whatever the batch entry and head:
                    if (s == 0) {                              // loaded once (also where the first head needs nothing)
                        raw.scw[0][0] = kvc_load_at<uint32_t>(a.scale + tk0, 4u * (uint32_t)lane);
                        raw.mnw[0][0] = kvc_load_at<uint16_t>(a.min_i8 + tk0, 2u * (uint32_t)lane);
                    } else {
                        raw.scw[s][0] = raw.scw[0][0];
                        raw.mnw[s][0] = raw.mnw[0][0];
                    }
                } else if (!((skip_x >> s) & 1) && (s == 0 || !LATE_SECOND)) {
                    kvc_fetch_separate_params(a, row, b, h, lane, s, raw);
                }
            }
#pragma unroll
            for (int r = 0; r < REP; r++) {
                if (EXPAND != 0 || ((skip_x >> s) & 1)) break;
                const int64_t xrow = (int64_t)b * a.q_heads + h * REP + r;
                if (KvcGeom<KIND>::SOFTMAX) {
                    const uint2 v = kvc_load_at<uint2>(a.scores + xrow * a.scores_stride + tk0, 8u * (uint32_t)lane);
                    raw.x[s][r][0] = v.x;
                    raw.x[s][r][KvcGeom<KIND>::XW - 1] = v.y;
                } else {
                    raw.x[s][r][0] = kvc_load_at<uint32_t>(a.x + xrow * a.tokens + tk0, 4u * (uint32_t)lane);
                }
            }
        }
    }
}

// The same for callers that know the tile by its row and column only.
template <int REP, int KIND, int EXPAND = 0>
__device__ __forceinline__ void kvc_fetch_tile(const KvcFusedArgs &a, int row, int col, uint32_t bi_off, uint32_t bi_bn,
                                               int lane, KvcRaw<REP, KvcGeom<KIND>::SLOTS, KvcGeom<KIND>::XW> &raw)
{
    kvc_fetch_tile<REP, KIND, EXPAND>(a, kvc_tile_pos<KIND == 0>(a, row, col), bi_off, bi_bn, lane, raw);
}

__device__ __forceinline__ float kvc_half_bits_to_float(uint32_t bits16)
{
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

// What the decode step needs to know about a staged tile.
struct KvcStaged {
    bool fits;            // staged in LDS (wave-uniform); otherwise decode from global memory
    uint32_t u0;          // fast-path start position (`lb` bits before the first code) in the lane's LDS words
    const uint32_t *gwords;   // the lane's stream in global memory, from the aligned word holding its first byte
    uint32_t gnwords, gpos;
};

// Move a fetched tile's payload into the wave's packed LDS area (least-significant-bit-first words, skewed if asked
// for) and work out where this lane's stream lies.  `first`: byte offset of the lane's stream in the packed area;
// `longest`: with per-lane rows, the longest lane stream of the tile in words.  The caller finishes st.u0.
template <class Raw>
__device__ __forceinline__ KvcStaged kvc_stage_payload(const KvcFusedArgs &a, int lane, const Raw &raw, uint32_t *pack,
                                                       uint32_t &first_out, uint32_t &longest_out)
{
    KvcStaged st;
    const uint32_t bn = raw.bn;
    // the previous lane's thread_info: one lane shift over the whole wave (lane 0 starts the tile)
    const uint32_t ti_prev = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.ti_cur, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
    uint32_t start = lane ? ti_prev >> 3 : 0u, end = raw.ti_cur >> 3;
    if (start > bn) start = bn;
    if (end > bn) end = bn;
    if (end < start) end = start;
    const uint8_t *src = a.s.enc + raw.off;
    const uint32_t head = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);
    const uint32_t nchunks = bn ? (head + bn + 15u) >> 4 : 0u;
    const uint32_t first = head + start;                                   // byte offset in the packed area
    const uint32_t nwords = end > start ? ((first & 3u) + (end - start) + 3u) >> 2 : 0u;
    {
        const uint8_t *lsrc = src + start;
        const uint32_t skew = (uint32_t)(reinterpret_cast<uintptr_t>(lsrc) & 3u);
        st.gwords = reinterpret_cast<const uint32_t *>(lsrc - skew);
        st.gnwords = nwords;
        st.gpos = skew * 8u;
    }
    // the packed area keeps row_words spare words at its end: the copy into rows moves the same
    // number of words for every lane, so the last lanes read past the payload
    bool fits = KVC_PACK_LEAD + 4u * nchunks + 3u + (uint32_t)a.row_words <= (uint32_t)a.pack_logical;
    uint32_t longest = 0;
    if (a.row_words) {
        longest = kvc_wave_max_dpp(nwords);
        fits = fits && longest + 3u <= (uint32_t)a.row_words;
    }
    st.fits = fits;
    st.u0 = 0;
    if (fits) {
        const uint32_t skew = (uint32_t)a.skew;
        // chunk c holds payload words 4c .. 4c + 3 (after the lead words); chunks never straddle a run of 32.
        // Chunk lane + 64 j lies a fixed number of words after chunk lane + 64 (j - 1), skewed or not, and whether
        // a chunk opens a run of 32 (and so is also the copy that ends the previous run) depends on the lane alone.
        const uint32_t w0 = KVC_PACK_LEAD + 4u * (uint32_t)lane;
        uint32_t *dst0 = pack + kvc_skewed(w0, skew);
        const uint32_t jstride = 256u + 8u * skew;
        const bool opens_run = skew && (w0 & 31u) == 0u;
        auto put = [&](uint32_t *dstw, uint4 v) {
            v.x = kvc_stream_word(v.x);
            v.y = kvc_stream_word(v.y);
            v.z = kvc_stream_word(v.z);
            v.w = kvc_stream_word(v.w);
            uint2 *dst = reinterpret_cast<uint2 *>(dstw);                            // 8-byte aligned either way
            dst[0] = make_uint2(v.x, v.y);
            dst[1] = make_uint2(v.z, v.w);
            if (opens_run) dst[-1] = make_uint2(v.x, v.y);
        };
#pragma unroll
        for (int j = 0; j < KVC_PRE_CHUNKS; j++) {
            const uint32_t c = (uint32_t)lane + 64u * j;
            if (c < nchunks) put(dst0 + j * jstride, raw.pay[j]);
        }
        const uint8_t *g = src - head;
        for (uint32_t c = (uint32_t)lane + 64u * KVC_PRE_CHUNKS; c < nchunks; c += KVC_WAVE)            // tiles beyond 4 KiB
            put(dst0 + (c >> 6) * jstride, kvc_load_at<uint4>(g, 16u * c));
    }
    first_out = first;
    longest_out = longest;
    return st;
}

// ---------------------------------------------------------------------------------------------------
// matrix-core variant (kvc_fused_mfma_impl.h)
// ---------------------------------------------------------------------------------------------------
// Columns of the operand matrix: every query head contributes a high and a low fp16 part of its weight, four
// columns per v_mfma_f32_4x4x4_16b_f16.
constexpr int kvc_mfma_sets(int rep) { return (2 * rep + 3) / 4; }
constexpr int KVC_MFMA_GROUPS = 32;       // groups of four elements per lane stream (128 / 4)
// LDS words per wave for the operand tables of one tile: per head slot 32 groups x sets x (4 columns x 4 fp16), and
// in rounded mode 32 groups x {two min pairs, two scale pairs}
constexpr int kvc_mfma_ops_words(int slots, int rep, bool rounded)
{
    return slots * (KVC_MFMA_GROUPS * kvc_mfma_sets(rep) * 8 + (rounded ? KVC_MFMA_GROUPS * 4 : 0));
}
void kvc_launch_fused_mfma(int rep, int kind, bool rounded, const KvcFusedArgs &a, dim3 grid, size_t lds, hipStream_t stream);
