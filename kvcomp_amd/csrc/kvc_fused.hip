// kvc_fused.hip -- Huffman decode fused with the two matvecs of decode attention: decoded symbols go
// from the LDS lookup straight into an fp32 FMA and never reach HBM.
//
//   kvc_fused_kernel<REP, 0>      <- huffman_decode_and_mat_vec_mul   (kvcomp_cuda_extension/src/kernels.cu:721-776)
//   kvc_fused_kernel<REP, 1 .. 4> <- v_huffman_decode_and_mat_vec_mul (kernels.cu:778-861); 3 / 4 form the softmax
//                                    weights of each 128-token group from raw scores on the fly
//   kvc_expand_kernel<KIND, DEQ>  <- huffman_decode / v_huffman_decode (kernels.cu:602-719) on the same pipeline
//   kvc_attention_decode          one call per layer: fused K, fused V, merge (+ the fp16 tails)
//
// One wave64 per tile, lane t owns stream t (K: a token, V: a channel), exactly the reference's work split.
// Every lane decodes one symbol (or exactly two, with the pair table) per step, so step i means "channel i" (K)
// or "token i of the 128-token group" (V) for the whole wave and the other FMA operand is wave-uniform:
//   K: score  = sum_i (sym_i + min_i) scale_i q_i = sum_i sym_i q'_i + sum_i min_i q'_i,  q'_i = scale_i q_i
//   V: out_d  = sum_t (sym_t + min_t) scale_t p_t = sum_t sym_t w_t  + sum_t min_t w_t,   w_t  = scale_t p_t
// q' / w are computed once per tile into an operand table in LDS; lane l reads element 4k + (l & 3) of every
// block of four and the FMA picks its operand from the right lane of the quad (a DPP modifier, no instruction).
// REP query heads share one KV head (grouped-query attention): the tile is decoded once and feeds REP accumulators.
//
// Pipeline per wave: everything a tile needs from global memory is fetched into registers one tile ahead;
// staging converts the payload to least-significant-bit-first words in LDS (optionally with two spare words per
// 32, which spreads lanes that would otherwise share a bank), builds the operand table and reduces the constant
// term with DPP steps.
//
// Inner loop (the "fast" path, codes no longer than the table index):
//   window  32 stream bits, least significant first, held two bits up: the next `lbits` bits sit at bits
//           [lbits+1 : 2], so masking gives the byte offset of the table entry directly
//   entry   fp32 bit pattern of the symbol with the code length in its lowest mantissa byte: it is the FMA
//           operand as it stands, and as a shift count it rotates the window right by len (v_alignbit)
//   refill  64 stream bits (three words, two funnel shifts): G symbols from the low half, the window re-formed
//           from the register pair at the bits consumed, G more; G = what a 30-bit window is sure to hold
//           (30 / longest code, at most 8); the entries are summed and the low byte of the sum is the number
//           of bits consumed
//   pairs   with codes of at most 4 bits a table of 8-byte entries yields two symbols per look-up
// Codebooks whose average code is short may use a larger G than is safe; lanes then note the largest
// consumption they saw, and if any lane went over, the wave decodes that tile again on the slow path.
//
// Slow path (codebooks with codes longer than the table index, tiles larger than the staging area, or
// the rare overflow above): one symbol per refill, generic table read from global memory, payload read
// from LDS or -- for an oversized tile -- from global memory.
#include "kvc_fused_common.h"

// -- slow path ----------------------------------------------------------------------------------------
// One symbol per refill; table and long-code list in global memory; words from LDS (staged, bit-reversed)
// or from global memory (raw, bounds-checked word by word).
// Returns sum_i sym_i * ops[i * REP + r] for each query head r (ops: this lane's operand table in LDS).
template <int REP, bool GSRC>
__device__ __noinline__ KvcVec<REP> kvc_slow_tile(const uint32_t *words, uint32_t nwords, uint32_t pos,
                                                  const uint32_t *__restrict__ lut_g, int n, const float *ops,
                                                  uint32_t skew, bool rounded)
{
    const uint32_t lshift = 32u - lut_g[0], nlong = lut_g[2];
    const uint32_t *longs = lut_g + KVC_LUT_HEADER_WORDS;
    const uint32_t *entries = lut_g + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    KvcVec<REP> acc;
#pragma unroll
    for (int r = 0; r < REP; r++) acc.v[r] = 0.f;
    for (int i = 0; i < n; i++) {
        const uint32_t wi = pos >> 5;
        uint32_t w0 = 0, w1 = 0;
        // either way the first stream bit of a word ends up in the most significant bit
        if (wi < nwords) w0 = GSRC ? kvc_bswap(words[wi]) : __brev(words[kvc_skewed(wi, skew)]);
        if (wi + 1 < nwords) w1 = GSRC ? kvc_bswap(words[wi + 1]) : __brev(words[kvc_skewed(wi + 1, skew)]);
        const uint32_t hi = (uint32_t)(((((uint64_t)w0) << 32 | w1) << (pos & 31u)) >> 32);
        const uint32_t e = entries[hi >> lshift];
        uint32_t len = e & 0xffu, sym = (e >> 8) & 0xffu;
        if (len == 0) {
            len = 1;
            sym = 0;
            for (uint32_t j = 0; j < nlong; j++) {
                const uint32_t c = longs[2 * j], ls = longs[2 * j + 1];
                const uint32_t l = ls & 0xffu;
                if (((hi ^ c) >> (32u - l)) == 0u) {
                    len = l;
                    sym = (ls >> 8) & 0xffu;
                    break;
                }
            }
        }
        const float f = (float)sym;
        if (rounded) {
            const float *o = ops + i * (REP + 1);
            const float v = kvc_rounded_value(__float2half_rn(f), __float_as_uint(o[0]));
#pragma unroll
            for (int r = 0; r < REP; r++) acc.v[r] = fmaf(v, o[1 + r], acc.v[r]);
        } else {
#pragma unroll
            for (int r = 0; r < REP; r++) acc.v[r] = fmaf(f, ops[i * REP + r], acc.v[r]);
        }
        pos += len;
    }
    return acc;
}

// -- fast path ----------------------------------------------------------------------------------------
// n symbols (a multiple of G) from bit u + 2 of the staged words on; acc[r] += sym_i * ops[i * REP + r].
// `ops` is this lane's view of the wave's operand table in LDS: the same address in every lane (a broadcast
// read) except in V tiles that straddle two heads, where the lanes of the second head point at its table.
// Returns through `u` the new position and through `worst` the largest number of bits a group consumed.

// acc += x * (the value of `quad` in lane (l & ~3) + J of lane l's quad): the lane permute rides on the FMA's
// first operand, so picking one of the four operands a quad holds costs no instruction of its own.
// (`quad` comes straight from an LDS read and `acc` is not the permuted operand, so no VALU-write -> permuted-read
// hazard can arise between consecutive FMAs.)  The inline assembly is opaque to the compiler's hazard recogniser, so it
// has a twin (BUILTIN) that expresses the same permute through the compiler's own intrinsic and leaves instruction
// selection and hazard handling to it; KvcFusedArgs::builtin_dpp selects it, and a test holds the two to equal bits.
template <int J, bool BUILTIN>
__device__ __forceinline__ void kvc_fma_quad_pick(float &acc, uint32_t quad, float x)
{
    if (BUILTIN) {
        const int picked = __builtin_amdgcn_update_dpp(0, (int)quad, J * 0x55 /* quad_perm:[J,J,J,J] */, 0xf, 0xf, false);
        acc = fmaf(__int_as_float(picked), x, acc);
    } else {
        asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[%3,%3,%3,%3] row_mask:0xf bank_mask:0xf"
            : "+v"(acc)
            : "v"(quad), "v"(x), "n"(J));
    }
}

template <int G, bool CHECK, bool SKEW, int REP, bool BUILTIN>
__device__ __forceinline__ void kvc_fast_dot(const uint32_t *stage, uint32_t &u,
                                             uint32_t fentry_base, uint32_t mask4, int n,
                                             const float *ops, float (&acc)[REP], uint32_t &worst)
{
    const float *ops_q = ops + (__lane_id() & 3);
    const uint32_t sbase = (uint32_t)(uintptr_t)(const kvc_lds_word *)stage;
    for (int i = 0; i < n; i += G) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1];
        // The group's G * REP operands, four per register: lane l holds element l & 3 of each block of four
        // and the FMA picks its operand from the right lane of the quad.  One 4-byte read per lane moves a
        // quarter of what a 16-byte broadcast read of the same four values would.
        constexpr int NBLK = (G * REP + 3) / 4;
        uint32_t blk[NBLK];
#pragma unroll
        for (int k = 0; k < NBLK; k++) blk[k] = __float_as_uint(ops_q[i * REP + 4 * k]);
        // 32 stream bits from bit u on: bits [1:0] are the pair before the lane's position, the next code
        // starts at bit 2
        uint32_t R = __builtin_amdgcn_alignbit(w1, w0, u);
        uint32_t es = 0;
        kvc_static_for<G>([&](auto g_) {
            constexpr int g = decltype(g_)::value;
            const uint32_t e = *(const kvc_lds_u32 *)(uintptr_t)((R & mask4) | fentry_base);
            R = __builtin_amdgcn_alignbit(R, R, e);                   // rotate right by len
            es += e;
            const float f = __uint_as_float(e);
            kvc_static_for<REP>([&](auto r_) {
                constexpr int r = decltype(r_)::value;
                constexpr int k = g * REP + r;
                kvc_fma_quad_pick<k & 3, BUILTIN>(acc[r], blk[k >> 2], f);
            });
        });
        const uint32_t used = es & 0xffu;
        if (CHECK) worst = used > worst ? used : worst;
        u += used;
    }
}

// The same with 64 stream bits per refill from LDS: G symbols are decoded from the low word, the window is
// re-formed from the register pair at the bits consumed so far (fewer than 32 unless the group overflowed, which
// `worst` reports), G more follow.  Halves the refills (address arithmetic, LDS round trip, length sums) per symbol.
template <int G, bool CHECK, bool SKEW, int REP, bool BUILTIN>
__device__ __forceinline__ void kvc_fast_dot2(const uint32_t *stage, uint32_t &u,
                                              uint32_t fentry_base, uint32_t mask4, int n,
                                              const float *ops, float (&acc)[REP], uint32_t &worst)
{
    const float *ops_q = ops + (__lane_id() & 3);
    const uint32_t sbase = (uint32_t)(uintptr_t)(const kvc_lds_word *)stage;
    for (int i = 0; i < n; i += 2 * G) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        constexpr int NBLK = (2 * G * REP + 3) / 4;
        uint32_t blk[NBLK];
#pragma unroll
        for (int k = 0; k < NBLK; k++) blk[k] = __float_as_uint(ops_q[i * REP + 4 * k]);
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0, used1 = 0;
        kvc_static_for<2 * G>([&](auto g_) {
            constexpr int g = decltype(g_)::value;
            if (g == G) {
                if (CHECK) used1 = es & 0xffu;
                R = __builtin_amdgcn_alignbit(hi, lo, es);
            }
            const uint32_t e = *(const kvc_lds_u32 *)(uintptr_t)((R & mask4) | fentry_base);
            if (g != G - 1 && g != 2 * G - 1) R = __builtin_amdgcn_alignbit(R, R, e);
            es += e;
            const float f = __uint_as_float(e);
            kvc_static_for<REP>([&](auto r_) {
                constexpr int r = decltype(r_)::value;
                constexpr int k = g * REP + r;
                kvc_fma_quad_pick<k & 3, BUILTIN>(acc[r], blk[k >> 2], f);
            });
        });
        const uint32_t used = es & 0xffu;
        if (CHECK) {
            const uint32_t used2 = used - used1;
            const uint32_t m = used1 > used2 ? used1 : used2;
            worst = m > worst ? m : worst;
        }
        u += used;
    }
}

// Rounded mode: the dequantized value is rounded to fp16 before the multiplication (see KvcFusedArgs::rounded).
// 64 stream bits per refill, four symbols from each half (codes of at most 7 bits).  The table entries carry the
// symbol as fp16 in their upper half (and the length in the lowest byte); element i's {min, scale} (two fp16 in
// one word) and weights come from one address for the whole wave.
template <bool SKEW, int REP>
__device__ __forceinline__ void kvc_rounded_dot(const uint32_t *stage, uint32_t &u, uint32_t fentry_base, uint32_t mask4,
                                                int n, const float *ops, float (&acc)[REP])
{
    constexpr int OPS = REP + 1;
    const uint32_t sbase = (uint32_t)(uintptr_t)(const kvc_lds_word *)stage;
    for (int i = 0; i < n; i += 8) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0;
        kvc_static_for<8>([&](auto g_) {
            constexpr int g = decltype(g_)::value;
            if (g == 4) R = __builtin_amdgcn_alignbit(hi, lo, es);        // at most 28 bits consumed so far
            const uint32_t e = *(const kvc_lds_u32 *)(uintptr_t)((R & mask4) | fentry_base);
            if (g != 3 && g != 7) R = __builtin_amdgcn_alignbit(R, R, e);
            es += e;                                                       // only the lowest byte is read below
            const float *o = ops + (i + g) * OPS;
            const float v = kvc_rounded_value(__ushort_as_half((unsigned short)(e >> 16)), __float_as_uint(o[0]));
#pragma unroll
            for (int r = 0; r < REP; r++) acc[r] = fmaf(v, o[1 + r], acc[r]);
        });
        u += es & 0xffu;
    }
}

// Two symbols per look-up.  When twice the longest code fits the index, every index decodes to exactly two
// symbols, so the lanes stay in step (step j of the wave = elements 2j and 2j + 1) while the look-ups, window
// shifts and length sums per symbol halve.  An entry is two words: the first symbol's fp32 pattern with the
// length of BOTH codes in its lowest mantissa byte, then the second symbol's fp32 pattern.  Entries are
// 8 bytes, so the window is held three bits up (look-behind of three) and "window bits & mask" is the
// entry's byte offset.  One refill from LDS fetches 64 stream bits: two pairs are decoded from the low
// word, the window is re-formed from the register pair at the bits consumed, two more pairs follow.
typedef uint32_t kvc_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) kvc_u32x2 kvc_lds_u32x2;

template <bool SKEW, int REP, bool BUILTIN>
__device__ __forceinline__ void kvc_pair_dot(const uint32_t *stage, uint32_t &u, uint32_t mask8,
                                             uint32_t table_base, int n, const float *ops, float (&acc)[REP])
{
    const float *ops_q = ops + (__lane_id() & 3);
    const uint32_t sbase = (uint32_t)(uintptr_t)(const kvc_lds_word *)stage;
    for (int i = 0; i < n; i += 8) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        constexpr int NBLK = 2 * REP;                                   // 8 symbols x REP operands, four per register
        uint32_t blk[NBLK];
#pragma unroll
        for (int k = 0; k < NBLK; k++) blk[k] = __float_as_uint(ops_q[i * REP + 4 * k]);
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0;
        kvc_static_for<4>([&](auto p_) {
            constexpr int p = decltype(p_)::value;
            if (p == 2) R = __builtin_amdgcn_alignbit(hi, lo, es);      // <= 24 bits consumed so far
            const kvc_u32x2 e = *(const kvc_lds_u32x2 *)(uintptr_t)((R & mask8) | table_base);
            if (p != 1 && p != 3) R = __builtin_amdgcn_alignbit(R, R, e.x);
            es += e.x;
            kvc_static_for<REP>([&](auto r_) {
                constexpr int r = decltype(r_)::value;
                constexpr int k0 = (2 * p) * REP + r, k1 = (2 * p + 1) * REP + r;
                kvc_fma_quad_pick<k0 & 3, BUILTIN>(acc[r], blk[k0 >> 2], __uint_as_float(e.x));
                kvc_fma_quad_pick<k1 & 3, BUILTIN>(acc[r], blk[k1 >> 2], __uint_as_float(e.y));
            });
        });
        u += es & 0xffu;
    }
}

// Move a fetched tile into LDS: payload -> packed area (-> per-lane rows), operands -> table; returns the
// constant terms sum_i min_i * operand_i in bias[].
template <int REP, int KIND, int EXPAND = 0>
__device__ __forceinline__ KvcStaged kvc_stage_tile(const KvcFusedArgs &a, int row, int col, int lane,
                                                    const KvcRaw<REP, KvcGeom<KIND>::SLOTS, KvcGeom<KIND>::XW> &raw, float *ops,
                                                    uint32_t *pack, uint32_t *rows, float (&bias)[REP], int &sel_out,
                                                    uint32_t lb)
{
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    const int D = a.head_dim;
    uint32_t first, longest;
    KvcStaged st = kvc_stage_payload(a, lane, raw, pack, first, longest);
    const bool fits = st.fits;
    const int pmode = kvc_pair_mode<KIND>(a);
    // ---- operand table: element i of head slot s, query head r at ops[(s * 128 + i) * REP + r]
    float bias_s[SLOTS][REP];
    const bool straddles = SLOTS == 2 && (col * KVC_WAVE) % D + KVC_WAVE > D;      // wave-uniform
#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
#pragma unroll
        for (int r = 0; r < REP; r++) bias_s[s][r] = 0.f;
        if (s == 1 && !straddles) continue;                    // no lane of this tile belongs to a second head
        const bool live = KIND != 0 || 2 * lane < D;
        if (EXPAND == 1) continue;
        if (EXPAND == 2) {                           // element i of slot s -> {min, scale} as two fp16 at ops[s * 128 + i]
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int i = 2 * lane + half;
                const uint32_t mn_h = __half_as_ushort(__float2half_rn((float)raw.min_int(s, half, pmode)));   // exact
                ops[s * 128 + i] = __uint_as_float(mn_h | ((live ? raw.scale_bits(s, half, pmode) : 0u) << 16));
            }
            continue;
        }
        float wgt[REP][2];                           // the two elements' weights: q, p, or exp(score - max)
#pragma unroll
        for (int r = 0; r < REP; r++) {
            if (KvcGeom<KIND>::SOFTMAX) {
                const float s0 = __uint_as_float(raw.x[s][r][0]) * a.sm_scale;
                const float s1 = __uint_as_float(raw.x[s][r][KvcGeom<KIND>::XW - 1]) * a.sm_scale;
                const float m = kvc_wave_fmax_dpp(fmaxf(s0, s1));
                wgt[r][0] = __expf(s0 - m);
                wgt[r][1] = __expf(s1 - m);
                const float l = kvc_wave_sum_dpp(wgt[r][0] + wgt[r][1]);
                if (lane == 0) {
                    int bh = (col * KVC_WAVE) / D + s;
                    const int bh_max = a.batch * a.kv_heads - 1;
                    bh = bh < bh_max ? bh : bh_max;
                    const int b = bh / a.kv_heads, h = bh - b * a.kv_heads;
                    float *ml = a.ml + (((int64_t)row * a.batch + b) * a.q_heads + h * REP + r) * 2;
                    ml[0] = m;     // tiles that share a head write the same pair
                    ml[1] = l;
                }
            } else {
                wgt[r][0] = kvc_half_bits_to_float(raw.x[s][r][0] & 0xffffu);
                wgt[r][1] = kvc_half_bits_to_float(raw.x[s][r][0] >> 16);
            }
        }
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int i = 2 * lane + half;
            const float sc = live ? kvc_half_bits_to_float(raw.scale_bits(s, half, pmode)) : 0.f;
            const float mn = (float)raw.min_int(s, half, pmode);
            if (a.rounded) {                             // wave-uniform
                float *o = ops + (s * 128 + i) * (REP + 1);
                const uint32_t mn_h = __half_as_ushort(__float2half_rn(mn));                  // exact
                o[0] = __uint_as_float(mn_h | ((live ? raw.scale_bits(s, half, pmode) : 0u) << 16));
#pragma unroll
                for (int r = 0; r < REP; r++) o[1 + r] = wgt[r][half];
                continue;
            }
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const float v = sc * wgt[r][half];
                ops[(s * 128 + i) * REP + r] = v;
                bias_s[s][r] += mn * v;
            }
        }
#pragma unroll
        for (int r = 0; r < REP; r++) bias_s[s][r] = kvc_wave_sum_dpp(bias_s[s][r]);
    }
    int sel = 0;
    if (SLOTS == 2) {
        const int c0 = col * KVC_WAVE;
        sel = (c0 % D + lane) >= D;                                        // 1 past a head boundary
    }
    sel_out = sel;
#pragma unroll
    for (int r = 0; r < REP; r++) bias[r] = (SLOTS == 2 && sel) ? bias_s[SLOTS - 1][r] : bias_s[0][r];
    kvc_wave_sync();
    // ---- per-lane rows: [lead word][the words of the packed area that hold this lane's stream]
    // Rows are an odd number of words apart, so lanes that are equally deep into their streams read 64
    // different addresses spread evenly over the banks; in the packed area such lanes sit one stream length
    // apart, which lines them up on a few banks whenever that length is close to a divisor of the bank count.
    if (fits) {
        const uint32_t w0 = KVC_PACK_LEAD + (first >> 2);
        if (a.row_words) {
            uint32_t *my_row = rows + lane * a.row_words + 1;
            const uint32_t *my_pack = pack + w0;
            // the same (even) number of words for every lane; what a lane copies beyond its own stream is
            // never decoded.  Rows hold an even number of words after the lead word.
            for (uint32_t k = 0; k < longest; k += 2) {
                const uint32_t wa = my_pack[k], wb = my_pack[k + 1];
                my_row[k] = wa;
                my_row[k + 1] = wb;
            }
            st.u0 = 32u + (first & 3u) * 8u - lb;
            kvc_wave_sync();
        } else {
            st.u0 = 32u * KVC_PACK_LEAD + first * 8u - lb;
        }
    } else {
        st.u0 = 0;
    }
    return st;
}

template <int REP, int KIND>
__global__ void __launch_bounds__(KVC_WG, KVC_FUSED_OCC(REP, KIND)) kvc_fused_kernel(KvcFusedArgs a)
{
    constexpr bool IS_K = KIND == 0;
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    // dynamic LDS: the fused table (at offset 0, so that its address folds into the lookups), then per wave:
    // operand table, packed payload, rows
    extern __shared__ __align__(16) uint32_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int D = a.head_dim;
    const int ops_per_elem = a.rounded ? REP + 1 : REP;
    const int per_wave = SLOTS * 128 * ops_per_elem + a.pack_words + KVC_WAVE * a.row_words;
    uint32_t *s_fentry = smem;
    float *ops = reinterpret_cast<float *>(smem + a.table_words + wave * per_wave);
    uint32_t *pack = smem + a.table_words + wave * per_wave + SLOTS * 128 * ops_per_elem;
    uint32_t *rows = pack + a.pack_words;
    const int row = blockIdx.y;
    const int64_t cb = a.s.rows_per_codebook ? row / a.s.rows_per_codebook : 0;
    const uint32_t *__restrict__ lut_g = a.s.luts + cb * KVC_LUT_WORDS;
    const uint32_t lbits = lut_g[0], nlong = lut_g[2];
    const bool fast_book = nlong == 0 && lbits <= (uint32_t)KVC_LUT_MAX_BITS && (1u << lbits) <= (uint32_t)a.table_words;
    // table entries as the fast loops use them: a length beyond the index width (possible only in a table that
    // kvc_build_lut did not write) is cut down, which bounds how far a lane's position can run (see
    // kvc_refill_address)
    auto fentry = [&](uint32_t i) {
        const uint32_t e = lut_g[KVC_LUT_FENTRY_OFFSET + i];
        return (e & 0xffu) > lbits ? (e & ~0xffu) | lbits : e;
    };
    // two symbols per look-up when every pair of codes fits the pair table's index
    const uint32_t pbits = 2u * lut_g[1];
    const bool pairs = fast_book && !a.rounded && a.pair_bits != 0 && pbits <= (uint32_t)a.pair_bits && lbits <= 7u;
    if (pairs) {
        // the single-symbol table goes to the (not yet used) per-wave areas, the pair table is derived from it
        uint32_t *tmp = smem + a.table_words;
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) tmp[i] = fentry(i);
        __syncthreads();
        const uint32_t m1 = (1u << lbits) - 1u;
        for (uint32_t idx = tid; idx < (1u << pbits); idx += KVC_WG) {
            const uint32_t e0 = tmp[idx & m1];
            const uint32_t e1 = tmp[(idx >> (e0 & 0xffu)) & m1];
            smem[2 * idx] = e0 + (e1 & 0xffu);           // both lengths; they sum to at most pbits < 256
            smem[2 * idx + 1] = e1;
        }
        __syncthreads();
    } else if (fast_book && a.rounded) {
        // the symbol as fp16 in the upper half of the entry, the length in its lowest byte
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) {
            const uint32_t e = fentry(i);
            const uint32_t sym_h = __half_as_ushort(__float2half_rn(__uint_as_float(e & 0xffffff00u)));
            s_fentry[i] = (sym_h << 16) | (e & 0xffu);
        }
    } else if (fast_book) {
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) s_fentry[i] = fentry(i);
    }
    const uint32_t lb = pairs ? 3u : 2u;                 // look-behind bits of the window = log2(entry bytes)
    if (lane < KVC_PACK_LEAD) pack[lane] = 0;
    if (a.row_words) rows[lane * a.row_words] = 0;
    __syncthreads();
    const uint32_t mask4 = ((1u << lbits) - 1u) << 2;
    const uint32_t fgroup = lut_g[4], fcheck = lut_g[5];
    const int n = IS_K ? D : KVC_V_TOKENS;                             // symbols per lane stream
    // 64 stream bits per refill: `fgroup` symbols from each half.  The main part takes as many refills of
    // 2 * fgroup symbols as leave a multiple of 8, the rest goes four per half.
    const bool dwin = a.double_window != 0 && fgroup >= 4 && n % 8 == 0;
    int n_main = 0;
    if (dwin) {
        const int per = 2 * (int)(fgroup > 8u ? 8u : fgroup);
        int k = n / per;
        while ((n - k * per) % 8 != 0) k--;
        n_main = k * per;
    }
    const uint32_t fe = (uint32_t)(uintptr_t)(kvc_lds_u32 *)s_fentry;  // 0: the table opens the dynamic LDS

    // this wave's tiles: T consecutive columns of one tile row
    const int T = a.s.tiles_per_wave;
    const int col0 = (blockIdx.x * KVC_WAVES_PER_WG + wave) * T;
    int ntiles = a.s.cols - col0;
    ntiles = ntiles < T ? ntiles : T;
    if (ntiles <= 0) return;
    // block_info of tile col0 + j in lane j
    uint32_t bi_off = 0, bi_bn = 0;
    if (lane < ntiles) {
        const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.s.block_infos + 8 * ((int64_t)row * a.s.cols + col0 + lane));
        bi_off = bi[0];
        bi_bn = bi[1];
    }
    KvcRaw<REP, SLOTS, KvcGeom<KIND>::XW> raw;
    kvc_fetch_tile<REP, KIND>(a, row, col0, __builtin_amdgcn_readlane(bi_off, 0), __builtin_amdgcn_readlane(bi_bn, 0), lane, raw);
    float bias[REP];
    int sel = 0;
    KvcStaged st = kvc_stage_tile<REP, KIND>(a, row, col0, lane, raw, ops, pack, rows, bias, sel, lb);
    for (int it = 0; it < ntiles; it++) {
        const int col = col0 + it;
        const bool more = it + 1 < ntiles;
        // The lane number is made opaque per tile: otherwise every address the fetch and the staging derive from
        // it is hoisted out of this loop and held in a register of its own through the decode loops (some twenty
        // registers, i.e. two waves per SIMD less)
        int lane_f = lane;
        asm volatile("" : "+v"(lane_f));
        if (more)   // loads for the next tile fly while this one is decoded
            kvc_fetch_tile<REP, KIND>(a, row, col + 1, __builtin_amdgcn_readlane(bi_off, it + 1),
                                      __builtin_amdgcn_readlane(bi_bn, it + 1), lane_f, raw);
        const float *my_ops = ops + sel * 128 * ops_per_elem;
        float acc[REP];
#pragma unroll
        for (int r = 0; r < REP; r++) acc[r] = 0.f;
        bool redo = !(fast_book && st.fits) || (a.rounded && lut_g[1] > 7u);
        if (!redo && a.rounded) {
            const uint32_t *words = a.row_words ? rows + lane * a.row_words : pack;
            uint32_t u = st.u0;
            if (!a.row_words && a.skew) kvc_rounded_dot<true, REP>(words, u, fe, mask4, n, my_ops, acc);
            else kvc_rounded_dot<false, REP>(words, u, fe, mask4, n, my_ops, acc);
        } else if (!redo) {
            const uint32_t *words = a.row_words ? rows + lane * a.row_words : pack;
            const bool skew = !a.row_words && a.skew;
            uint32_t u = st.u0, worst = 0;
            auto run = [&](auto skew_, auto builtin_) {
                constexpr bool SK = decltype(skew_)::value, BI = decltype(builtin_)::value;
                if (pairs) {
                    kvc_pair_dot<SK, REP, BI>(words, u, ((1u << pbits) - 1u) << 3, fe, n, my_ops, acc);
                } else if (dwin && !fcheck) {
                    if (fgroup >= 8) kvc_fast_dot2<8, false, SK, REP, BI>(words, u, fe, mask4, n_main, my_ops, acc, worst);
                    else if (fgroup == 7) kvc_fast_dot2<7, false, SK, REP, BI>(words, u, fe, mask4, n_main, my_ops, acc, worst);
                    else if (fgroup == 6) kvc_fast_dot2<6, false, SK, REP, BI>(words, u, fe, mask4, n_main, my_ops, acc, worst);
                    else if (fgroup == 5) kvc_fast_dot2<5, false, SK, REP, BI>(words, u, fe, mask4, n_main, my_ops, acc, worst);
                    const int rest = fgroup == 4 ? n : n - n_main;
                    if (rest) kvc_fast_dot2<4, false, SK, REP, BI>(words, u, fe, mask4, rest, my_ops + (n - rest) * REP, acc, worst);
                } else if (dwin && fgroup >= 4 && fgroup < 8) {
                    kvc_fast_dot2<4, true, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                } else if (fgroup >= 8 && !fcheck) {
                    kvc_fast_dot<8, false, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                } else if (fgroup >= 8) {
                    kvc_fast_dot<8, true, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                } else if (fgroup >= 4 && !fcheck) {
                    kvc_fast_dot<4, false, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                } else if (fgroup >= 4) {
                    kvc_fast_dot<4, true, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                } else {
                    kvc_fast_dot<2, false, SK, REP, BI>(words, u, fe, mask4, n, my_ops, acc, worst);
                }
            };
            if (a.builtin_dpp) {
                if (skew) run(std::true_type{}, std::true_type{});
                else run(std::false_type{}, std::true_type{});
            } else {
                if (skew) run(std::true_type{}, std::false_type{});
                else run(std::false_type{}, std::false_type{});
            }
            redo = __any(worst > 30u);
        }
        if (redo) {
            KvcVec<REP> res;
            if (st.fits) {
                const uint32_t *words = a.row_words ? rows + lane * a.row_words : pack;
                const uint32_t nw = (uint32_t)(a.row_words ? a.row_words : a.pack_logical);
                res = kvc_slow_tile<REP, false>(words, nw, st.u0 + lb, lut_g, n, my_ops, a.row_words ? 0u : (uint32_t)a.skew, a.rounded != 0);
            } else {
                res = kvc_slow_tile<REP, true>(st.gwords, st.gnwords, st.gpos, lut_g, n, my_ops, 0u, a.rounded != 0);
            }
#pragma unroll
            for (int r = 0; r < REP; r++) acc[r] = res.v[r];
        }
        // ---- results
        int64_t out_base, out_step;
        if (IS_K) {
            const int b = col / a.kv_heads, h = col - b * a.kv_heads;
            out_base = ((int64_t)b * a.q_heads + h * REP) * a.out_stride + (int64_t)row * KVC_WAVE + lane;
            out_step = a.out_stride;
        } else {
            const int c0 = col * KVC_WAVE;
            const int bh0 = c0 / D, d0 = c0 - bh0 * D;                  // wave-uniform
            const int past = (SLOTS == 2 && d0 + lane >= D) ? 1 : 0;     // this lane's channel lies in the next head
            const int bh = bh0 + past, d = d0 + lane - past * D;
            const int b0 = bh0 / a.kv_heads, h0 = bh0 - b0 * a.kv_heads;
            const int wrap = (h0 + past == a.kv_heads) ? 1 : 0;         // ... which may be the first head of the next batch entry
            const int b = b0 + wrap, h = wrap ? 0 : h0 + past;
            (void)bh;
            out_base = (((int64_t)row * a.batch + b) * a.q_heads + h * REP) * D + d;
            out_step = D;
        }
#pragma unroll
        for (int r = 0; r < REP; r++) {
            const int64_t o = out_base + r * out_step;
            const float v = acc[r] + bias[r];
            if (a.out_f32) reinterpret_cast<float *>(a.out)[o] = v;
            else reinterpret_cast<__half *>(a.out)[o] = __float2half(v);
        }
        if (more) {
            kvc_wave_sync();     // every lane is done reading this tile's LDS data
            int lane_s = lane;
            asm volatile("" : "+v"(lane_s));
            st = kvc_stage_tile<REP, KIND>(a, row, col + 1, lane_s, raw, ops, pack, rows, bias, sel, lb);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// plain decode and decode + dequantize on the same machinery
//   <- huffman_decode / v_huffman_decode (kvcomp_cuda_extension/src/kernels.cu:602-719), and with DEQ also
//      the (sym + min) * scale that follows them (models/cache/kvcomp_encode.py:146,161)
// Tiles are fetched one ahead, staged and decoded exactly as in kvc_fused_kernel; instead of feeding an FMA,
// every symbol (or its dequantized fp16 value) goes to a 32-element output slab in LDS, which the wave
// copies out with 8- and 16-byte stores: 32 channels of the tile's 64 tokens (K), or 32 tokens of its 64
// channels (V).
// ---------------------------------------------------------------------------------------------------
// G symbols per half window, 2 G per refill; put(i, g, e) receives the index i of the refill's first element,
// the element's place g in the refill as a compile-time constant, and the table entry.
template <int G, bool SKEW, class Put>
__device__ __forceinline__ void kvc_fast_emit2(const uint32_t *stage, uint32_t &u, uint32_t fentry_base, uint32_t mask4,
                                               int i0, int n, Put &&put)
{
    const uint32_t sbase = (uint32_t)(uintptr_t)(const kvc_lds_word *)stage;
    for (int i = i0; i < i0 + n; i += 2 * G) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0;
        kvc_static_for<2 * G>([&](auto g_) {
            constexpr int g = decltype(g_)::value;
            if (g == G) R = __builtin_amdgcn_alignbit(hi, lo, es);
            const uint32_t e = *(const kvc_lds_u32 *)(uintptr_t)((R & mask4) | fentry_base);
            if (g != G - 1 && g != 2 * G - 1) R = __builtin_amdgcn_alignbit(R, R, e);
            es += e;
            put(i, g_, e);
        });
        u += es & 0xffu;
    }
}

// One symbol per refill, table and long-code list in global memory (codes beyond the table index, tiles
// that do not fit the staging area, windows that may overflow); put1(i, symbol as an fp32 pattern).
template <bool GSRC, class Put>
__device__ __forceinline__ void kvc_slow_emit(const uint32_t *words, uint32_t nwords, uint32_t &pos,
                                           const uint32_t *__restrict__ lut_g, int i0, int n, uint32_t skew, Put &&put1)
{
    const uint32_t lshift = 32u - lut_g[0], nlong = lut_g[2];
    const uint32_t *longs = lut_g + KVC_LUT_HEADER_WORDS;
    const uint32_t *entries = lut_g + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    for (int i = i0; i < i0 + n; i++) {
        const uint32_t wi = pos >> 5;
        uint32_t w0 = 0, w1 = 0;
        if (wi < nwords) w0 = GSRC ? kvc_bswap(words[wi]) : __brev(words[kvc_skewed(wi, skew)]);
        if (wi + 1 < nwords) w1 = GSRC ? kvc_bswap(words[wi + 1]) : __brev(words[kvc_skewed(wi + 1, skew)]);
        const uint32_t hi = (uint32_t)(((((uint64_t)w0) << 32 | w1) << (pos & 31u)) >> 32);
        const uint32_t e = entries[hi >> lshift];
        uint32_t len = e & 0xffu, sym = (e >> 8) & 0xffu;
        if (len == 0) {
            len = 1;
            sym = 0;
            for (uint32_t j = 0; j < nlong; j++) {
                const uint32_t c = longs[2 * j], ls = longs[2 * j + 1];
                const uint32_t l = ls & 0xffu;
                if (((hi ^ c) >> (32u - l)) == 0u) {
                    len = l;
                    sym = (ls >> 8) & 0xffu;
                    break;
                }
            }
        }
        put1(i, __float_as_uint((float)sym));
        pos += len;
    }
}

// Output slab of one wave, copied to global memory whenever it is full:
//   K: [64 tokens][SLAB channels], rows one 32-bit word longer than the 64 bytes they carry (so that the lanes'
//      rows start in all banks); a lane packs the elements of its own row in a register, one word at a time
//   V: [SLAB tokens][64 channels], dense; consecutive elements of a lane lie a row apart, so they are written singly
template <bool IS_K, bool DEQ>
struct KvcSlab {
    using elem = std::conditional_t<DEQ, uint16_t, uint8_t>;
    static constexpr int ESZ = (int)sizeof(elem);
    static constexpr int SLAB = IS_K ? 64 / ESZ : 32;          // elements per lane between two copies
    static constexpr int K_ROW_WORDS = 64 / 4 + 1;
    static constexpr int WORDS = IS_K ? 64 * K_ROW_WORDS : SLAB * 64 * ESZ / 4;
};

#ifndef KVC_EXPAND_OCC
#define KVC_EXPAND_OCC 1
#endif
template <int KIND, bool DEQ>
__global__ void __launch_bounds__(KVC_WG, KVC_EXPAND_OCC) kvc_expand_kernel(KvcFusedArgs a)
{
    constexpr bool IS_K = KIND == 0;
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    using S = KvcSlab<IS_K, DEQ>;
    using elem = typename S::elem;
    extern __shared__ __align__(16) uint32_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int D = a.head_dim;
    const int ops_words = DEQ ? SLOTS * 128 : 0;
    const int per_wave = ops_words + a.pack_words + KVC_WAVE * a.row_words + a.out_words;
    uint32_t *s_fentry = smem;
    float *ops = reinterpret_cast<float *>(smem + a.table_words + wave * per_wave);
    uint32_t *pack = smem + a.table_words + wave * per_wave + ops_words;
    uint32_t *rows = pack + a.pack_words;
    elem *slab = reinterpret_cast<elem *>(rows + KVC_WAVE * a.row_words);
    const int row = blockIdx.y;
    const int64_t cb = a.s.rows_per_codebook ? row / a.s.rows_per_codebook : 0;
    const uint32_t *__restrict__ lut_g = a.s.luts + cb * KVC_LUT_WORDS;
    const uint32_t lbits = lut_g[0], nlong = lut_g[2];
    const bool fast_book = nlong == 0 && lbits <= (uint32_t)KVC_LUT_MAX_BITS && (1u << lbits) <= (uint32_t)a.table_words;
    if (fast_book)
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) {
            uint32_t e = lut_g[KVC_LUT_FENTRY_OFFSET + i];
            e = (e & 0xffu) > lbits ? (e & ~0xffu) | lbits : e;
            // dequantizing: the symbol as fp16 in the upper half of the entry, the length in its lowest byte
            if (DEQ) e = ((uint32_t)__half_as_ushort(__float2half_rn(__uint_as_float(e & 0xffffff00u))) << 16) | (e & 0xffu);
            s_fentry[i] = e;
        }
    if (lane < KVC_PACK_LEAD) pack[lane] = 0;
    if (a.row_words) rows[lane * a.row_words] = 0;
    __syncthreads();
    const uint32_t mask4 = ((1u << lbits) - 1u) << 2;
    const int n = IS_K ? D : KVC_V_TOKENS;
    const uint32_t fe = (uint32_t)(uintptr_t)(kvc_lds_u32 *)s_fentry;
    const bool fast_loop = fast_book && lut_g[1] <= 7u && n % 8 == 0;     // four codes of <= 7 bits fit a half window
    const bool wide16 = DEQ || (D & 15) == 0;                 // K rows start on 16-byte boundaries
    const uint32_t lb = 2u;

    const int T = a.s.tiles_per_wave;
    const int col0 = (blockIdx.x * KVC_WAVES_PER_WG + wave) * T;
    int ntiles = a.s.cols - col0;
    ntiles = ntiles < T ? ntiles : T;
    if (ntiles <= 0) return;
    uint32_t bi_off = 0, bi_bn = 0;
    if (lane < ntiles) {
        const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.s.block_infos + 8 * ((int64_t)row * a.s.cols + col0 + lane));
        bi_off = bi[0];
        bi_bn = bi[1];
    }
    KvcRaw<1, SLOTS, 1> raw;
    kvc_fetch_tile<1, KIND, DEQ ? 2 : 1>(a, row, col0, __builtin_amdgcn_readlane(bi_off, 0), __builtin_amdgcn_readlane(bi_bn, 0), lane, raw);
    float bias[1];
    int sel = 0;
    KvcStaged st = kvc_stage_tile<1, KIND, DEQ ? 2 : 1>(a, row, col0, lane, raw, ops, pack, rows, bias, sel, lb);
    for (int it = 0; it < ntiles; it++) {
        const int col = col0 + it;
        const bool more = it + 1 < ntiles;
        int lane_f = lane;                       // opaque per tile, as in kvc_fused_kernel
        asm volatile("" : "+v"(lane_f));
        if (more)
            kvc_fetch_tile<1, KIND, DEQ ? 2 : 1>(a, row, col + 1, __builtin_amdgcn_readlane(bi_off, it + 1),
                                    __builtin_amdgcn_readlane(bi_bn, it + 1), lane_f, raw);
        const float *my_ops = ops + sel * 128;
        const bool fast = fast_loop && st.fits;
        const uint32_t *words = st.fits ? (a.row_words ? rows + lane * a.row_words : pack) : st.gwords;
        const uint32_t nw = st.fits ? (uint32_t)(a.row_words ? a.row_words : a.pack_logical) : st.gnwords;
        const bool skew = st.fits && !a.row_words && a.skew;
        uint32_t u = st.fits ? st.u0 : st.gpos;                 // fast: lb bits before the code; slow: at the code
        if (st.fits && !fast) u += lb;
        // the value of element i: the symbol itself, or RN16((symbol + min_i) * scale_i) (an exact fp16 sum and one
        // fp16 multiplication).  FAST: e is a table entry of this kernel; otherwise the symbol as an fp32 pattern.
        auto value = [&](int i, uint32_t e, bool from_table) -> uint32_t {
            if (DEQ) {
                const __half sym = from_table ? __ushort_as_half((unsigned short)(e >> 16)) : __float2half_rn(__uint_as_float(e));
                const uint32_t ms = __float_as_uint(my_ops[i]);
                const __half mn = __ushort_as_half((unsigned short)(ms & 0xffffu)), sc = __ushort_as_half((unsigned short)(ms >> 16));
                return (uint32_t)__half_as_ushort(__hmul(__hadd(sym, mn), sc));
            }
            return (uint32_t)__uint_as_float(e);                           // the low mantissa bits add less than one
        };
        uint32_t *slab_w = reinterpret_cast<uint32_t *>(slab);
        uint32_t cur = 0;
        // fast loop: element i + g of the lane, g known at compile time
        auto put = [&](int i, auto g_, uint32_t e) {
            constexpr int g = decltype(g_)::value;
            constexpr int PER = 4 / S::ESZ;                                // elements per word
            const uint32_t v = value(i + g, e, true);
            if (IS_K) {
                cur = (g % PER == 0) ? v : cur | (v << (8 * S::ESZ * (g % PER)));
                if (g % PER == PER - 1)
                    slab_w[lane * S::K_ROW_WORDS + ((i & (S::SLAB - 1)) + g) / PER] = cur;
            } else {
                slab[((i + g) & (S::SLAB - 1)) * KVC_WAVE + lane] = (elem)v;
            }
        };
        // slow loop: one element at a time
        auto put1 = [&](int i, uint32_t e) {
            const int j = i & (S::SLAB - 1);
            slab[IS_K ? lane * (S::K_ROW_WORDS * 4 / S::ESZ) + j : j * KVC_WAVE + lane] = (elem)value(i, e, false);
        };
        for (int i0 = 0; i0 < n; i0 += S::SLAB) {
            const int len = n - i0 < S::SLAB ? n - i0 : S::SLAB;
            if (fast) {
                if (skew) kvc_fast_emit2<4, true>(words, u, fe, mask4, i0, len, put);
                else kvc_fast_emit2<4, false>(words, u, fe, mask4, i0, len, put);
            } else if (st.fits) {
                kvc_slow_emit<false>(words, nw, u, lut_g, i0, len, skew ? (uint32_t)a.skew : 0u, put1);
            } else {
                kvc_slow_emit<true>(words, nw, u, lut_g, i0, len, 0u, put1);
            }
            kvc_wave_sync();
            // ---- copy the slab out, 16 bytes per lane and store
            constexpr int PER16 = 16 / S::ESZ;                             // elements per piece
            if (IS_K) {
                // rows of `len` elements (64 bytes when full): four lanes per row
                elem *out = reinterpret_cast<elem *>(a.out) + (int64_t)row * KVC_WAVE * a.s.stride + (int64_t)col * D + i0;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const int f = lane + KVC_WAVE * t, r = f >> 2, c = f & 3;
                    if (c * PER16 < len) {
                        const uint32_t *src = slab_w + r * S::K_ROW_WORDS + 4 * c;
                        uint4 v = make_uint4(src[0], src[1], src[2], src[3]);
                        elem *dst = out + (int64_t)r * a.s.stride + c * PER16;
                        if (wide16) {
                            *reinterpret_cast<uint4 *>(dst) = v;
                        } else {                                            // uint8 rows with head_dim % 16 == 8: 8-byte alignment only
                            *reinterpret_cast<uint2 *>(dst) = make_uint2(v.x, v.y);
                            if (c * PER16 + PER16 <= len) *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(v.z, v.w);
                        }
                    }
                }
            } else {
                constexpr int PIECES = KVC_WAVE / PER16;                    // pieces per row of 64 channels
                elem *out = reinterpret_cast<elem *>(a.out) + ((int64_t)row * KVC_V_TOKENS + i0) * a.s.stride + (int64_t)col * KVC_WAVE;
#pragma unroll
                for (int t = 0; t < S::SLAB * PIECES / KVC_WAVE; t++) {
                    const int f = lane + KVC_WAVE * t, r = f / PIECES, c = f - r * PIECES;
                    if (r < len) {
                        const uint4 v = *reinterpret_cast<const uint4 *>(slab + r * KVC_WAVE + c * PER16);
                        *reinterpret_cast<uint4 *>(out + (int64_t)r * a.s.stride + c * PER16) = v;
                    }
                }
            }
            kvc_wave_sync();
        }
        if (more) {
            int lane_s = lane;
            asm volatile("" : "+v"(lane_s));
            st = kvc_stage_tile<1, KIND, DEQ ? 2 : 1>(a, row, col + 1, lane_s, raw, ops, pack, rows, bias, sel, lb);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------
template <int REP>
static void kvc_launch_fused(int kind, const KvcFusedArgs &a, dim3 grid, size_t lds, hipStream_t stream)
{
    if (kind == 0) hipLaunchKernelGGL((kvc_fused_kernel<REP, 0>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 1) hipLaunchKernelGGL((kvc_fused_kernel<REP, 1>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 2) hipLaunchKernelGGL((kvc_fused_kernel<REP, 2>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 3) hipLaunchKernelGGL((kvc_fused_kernel<REP, 3>), grid, dim3(KVC_WG), lds, stream, a);
    else hipLaunchKernelGGL((kvc_fused_kernel<REP, 4>), grid, dim3(KVC_WG), lds, stream, a);
}

// LDS layout of one workgroup: the fused table, then per wave the operand table(s), the packed payload of
// one tile and (optionally) the per-lane rows.  Sized from the encoder's hints (largest tile payload,
// longest lane stream); without them from twice the payload's means.  Tiles that do not fit are decoded
// from global memory, so the sizes only affect speed.  Everything stays within 64 KiB per workgroup.
static size_t kvc_plan_lds(KvcFusedArgs &a, int slots, int rep, int64_t encoded_bytes, int64_t tiles,
                           int64_t max_tile_bytes, int64_t max_stream_bytes, int max_code_bits, int64_t extra_words = 0,
                           bool allow_pairs = true, int64_t mfma_ops_words = 0)
{
    const int force_rows = kvc_option(KVC_OPT_FUSED_ROWS);   // 0 / 1 overrides the choice below
    a.table_words = 1 << ((max_code_bits >= 1 && max_code_bits <= KVC_LUT_MAX_BITS) ? max_code_bits : KVC_LUT_MAX_BITS);
    if (a.table_words < 4) a.table_words = 4;   // keeps the per-wave areas 16-byte aligned
    // room for the two-symbol table (8 bytes per index of 2 * longest-code bits) when the codes are short
    const int pair_limit = kvc_option(KVC_OPT_FUSED_PAIR_BITS);
    a.pair_bits = 0;
    a.rounded = 0;
    a.expand = 0;
    a.out_words = 0;
    a.double_window = kvc_option(KVC_OPT_FUSED_DOUBLE_WINDOW);
    a.builtin_dpp = kvc_option(KVC_OPT_FUSED_BUILTIN_DPP) != 0;
    a.half_table = kvc_option(KVC_OPT_FUSED_HALF_TABLE) != 0;
    if (allow_pairs && extra_words == 0 && max_code_bits >= 1 && 2 * max_code_bits <= pair_limit) {
        a.pair_bits = 2 * max_code_bits;
        // eight bytes per entry (fp32 symbols), four in the matrix-core kernels (fp16 symbols)
        const int words = (mfma_ops_words ? 1 : 2) << a.pair_bits;
        if (a.table_words < words) a.table_words = words;
    }
    // per wave, besides the payload
    const int64_t ops_words = mfma_ops_words ? mfma_ops_words : (int64_t)slots * 128 * rep + extra_words;
    const int64_t budget = (65536 / 4 - a.table_words - KVC_LDS_SLACK_WORDS) / KVC_WAVES_PER_WG - ops_words;   // words per wave
    const int64_t mean_tile = encoded_bytes / (tiles > 0 ? tiles : 1);
    // without the encoder's figure: tiles hold thousands of symbols, so their sizes stay close to the mean
    int64_t tile_bytes = max_tile_bytes > 0 ? max_tile_bytes : mean_tile + mean_tile / 4 + 256;
    if (tile_bytes > KVC_MAX_TILE_BYTES) tile_bytes = KVC_MAX_TILE_BYTES;
    // lead words + the payload's chunks (it may start anywhere in its first chunk) + look-ahead
    int64_t pack = KVC_PACK_LEAD + ((tile_bytes + 15 + 15) / 16) * 4 + 4;   // three look-ahead words, rounded up
    int64_t stream_bytes = max_stream_bytes > 0 ? max_stream_bytes : 2 * mean_tile / KVC_WAVE + 4;
    // lead word + the stream's words (it may start anywhere in its first word) + look-ahead, forced odd
    const int64_t row = ((stream_bytes + 3 + 3) / 4 + 3) | 1;
    const int64_t pack_rows = (pack + row + 3) / 4 * 4;      // spare words for the fixed-length copy into rows
    // Decoding from the plain packed payload lines the lanes up on a few banks when a small multiple of the mean
    // stream length is close to a multiple of the 32 banks (lane l reads about l mean-stream-lengths into the
    // payload).  The skewed layout cures that at the cost of 1/16 more LDS and two instructions per refill;
    // per-lane rows (an odd number of words apart) cure it too, but double the LDS a tile needs and cost a
    // copy, so they are only used when asked for.
    const double mean_stream_words = (double)encoded_bytes / (double)(tiles > 0 ? tiles : 1) / KVC_WAVE / 4.0;
    bool resonant = false;
    for (int k = 1; k <= 4; k++) {
        const double x = k * mean_stream_words / 32.0;
        const double dist = (x - (double)(int64_t)(x + 0.5)) * 32.0;
        if (x >= 0.5 && dist > -1.0 && dist < 1.0) resonant = true;
    }
    const bool use_rows = force_rows == 1 && pack_rows + KVC_WAVE * row <= budget;
    const int force_skew = kvc_option(KVC_OPT_FUSED_SKEW);
    const bool use_skew = !use_rows && (force_skew >= 0 ? force_skew != 0 : resonant);
    a.row_words = 0;
    a.skew = 0;
    if (use_rows) {
        a.row_words = (int)row;
        pack = pack_rows;
    }
    auto physical = [&](int64_t logical) { return use_skew ? (logical + 2 * (logical >> 5) + 2 + 3) / 4 * 4 : logical; };
    while (pack > 16 && physical(pack) > budget) pack -= 4;
    if (use_skew) a.skew = 2;
    a.pack_logical = (int)pack;
    a.pack_words = (int)physical(pack);
    return 4 * ((size_t)a.table_words + KVC_LDS_SLACK_WORDS +
                (size_t)KVC_WAVES_PER_WG * (size_t)(ops_words + a.pack_words + KVC_WAVE * a.row_words));
}

// Consecutive tiles of a row that one wave works through (fetching one ahead): as many as still leave
// every SIMD of the chip several waves.
constexpr int KVC_DEFAULT_SCHEDULE = 47020;      // runs of 4 for 70 % of the tiles, of 2 for 20 %, single tiles last
constexpr int KVC_DEFAULT_SCHEDULE_UNIT3 = 67020; // runs of 6 (two head pairs of head_dim 96), then of 3, single tiles last

// `unit`: V tiles (matrix-core kernels, rounded arithmetic) after which the heads repeat -- the tiles of one head, or of
// a pair of heads where head_dim is no multiple of 64 (three tiles over two heads of 96 channels): a wave that takes
// whole units builds every head's operand tables once.  0: nothing to share (K tiles; the other kernels).
static int kvc_plan_tiles_per_wave(int64_t tiles, int unit = 0, int rep = 1)
{
    const int forced_v = unit ? kvc_option(KVC_OPT_FUSED_TILES_PER_WAVE_V) : -1;
    const int forced = forced_v > 0 ? forced_v : kvc_option(KVC_OPT_FUSED_TILES_PER_WAVE);
    if (forced > 0) return forced > 64 ? 64 : forced;
    // measured on MI355X: two is best once there are enough tiles (the fetch of the second overlaps the
    // decode of the first; 49 152 tiles: 3 % faster than one); at 16 384 tiles one is 3 % faster, and longer runs
    // only leave fewer workgroups to balance over the chip (8 per wave: 15 % slower)
    // (V, 16 384 tiles of head_dim 128: with four query heads per KV head, whose four softmaxes and operand tables two
    // tiles of a head then share, 49.1 us for two per wave against 50.4 for one; with one query head 40.1 against 37.6)
    if (unit > 1 && unit <= 4 && forced_v < 0 && tiles >= 8192 && (rep >= 4 || tiles >= 32768)) return unit;
    return tiles >= 32768 ? 2 : 1;
}

// Schedule of a matrix-core launch over `tiles` tiles (see KvcFusedArgs::sched_*): long runs of tiles per wave
// first, so that most tiles share a wave's set-up and their fetches overlap the previous tile's decode, shorter ones
// after, single tiles last, so that the last workgroups to start are short.  Returns the number of workgroups, 0 for
// the plain 2-D grid.
static unsigned kvc_plan_schedule(KvcFusedArgs &a, int64_t tiles, int unit = 0, int rep = 1)
{
    a.sched_nseg = 0;
    int want = kvc_option(KVC_OPT_FUSED_SCHEDULE);
    if (unit && kvc_option(KVC_OPT_FUSED_SCHEDULE_V) >= 0) want = kvc_option(KVC_OPT_FUSED_SCHEDULE_V);
    if (want == 0 || a.s.rows_per_codebook != 0 || tiles > (int64_t)1 << 30) return 0;
    if (want < 0) {
        // few tiles: one or two per wave in the plain grid -- except V tiles of head_dim 128 with four or more query
        // heads per KV head, where a head's four softmaxes and operand tables are worth sharing between its two tiles and
        // the next head's: at 16 384 tiles, runs of 4 for half the tiles, 2 for 30 %, 1 for the rest 46.3 us, against 49.0
        // for two tiles per wave everywhere (with one query head: 38.7 against 36.2 for one tile per wave)
        const bool mid_v = unit == 2 && rep >= 4 && tiles >= 16384;
        if (tiles < 32768 && !mid_v) return 0;
        // runs that are whole units (and, halved and quartered, stay whole units or single tiles)
        want = tiles < 32768 ? 45030 : unit == 3 ? KVC_DEFAULT_SCHEDULE_UNIT3 : KVC_DEFAULT_SCHEDULE;
    }
    const int run0 = want / 10000, pct0 = (want / 100) % 100, pct1 = want % 100;
    if (run0 < 1 || run0 > 64 || pct0 + pct1 > 100) return 0;
    const int per_wg[KVC_SCHED_SEGMENTS] = {run0, run0 / 2 > 1 ? run0 / 2 : 1, run0 / 4 > 1 ? run0 / 4 : 1, 1};
    const int64_t rest = tiles - tiles * (pct0 + pct1) / 100;
    int64_t want_tiles[KVC_SCHED_SEGMENTS] = {tiles * pct0 / 100, tiles * pct1 / 100, rest / 2, 0};
    int64_t tile = 0, wg = 0;
    int k = 0;
    for (int i = 0; i < KVC_SCHED_SEGMENTS && tile < tiles; i++) {
        const int64_t chunk = (int64_t)per_wg[i] * KVC_WAVES_PER_WG;
        // whole workgroups; the last segment takes whatever is left
        int64_t n = i == KVC_SCHED_SEGMENTS - 1 ? tiles - tile : want_tiles[i] / chunk * chunk;
        if (n > tiles - tile) n = tiles - tile;
        if (n <= 0) continue;
        a.sched_run[k] = per_wg[i];
        a.sched_wg[k] = (int)wg;
        a.sched_tile[k] = (int)tile;
        tile += n;
        wg += (n + chunk - 1) / chunk;
        k++;
    }
    a.sched_nseg = k;
    for (int i = k; i <= KVC_SCHED_SEGMENTS; i++) {
        a.sched_wg[i] = (int)wg;
        a.sched_tile[i] = (int)tiles;
        if (i < KVC_SCHED_SEGMENTS) a.sched_run[i] = 1;
    }
    return (unsigned)wg;
}

// what the one-call attention adds to a plain fused launch
struct KvcFusedExtra {
    int64_t out_stride;          // K: row stride of the score matrix (0 = tokens)
    const float *scores;         // V: fp32 scores in place of p (softmax on the fly), or NULL
    int64_t scores_stride;
    float sm_scale;
    float *ml;
};

static int kvc_fused(int is_k, const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                     const uint8_t *d_block_infos, int64_t block_infos_bytes, const uint8_t *d_thread_infos,
                     int64_t thread_infos_bytes, const uint8_t *d_encoded, int64_t encoded_bytes,
                     const int8_t *d_min, const void *d_scale, int quant_mask, const void *d_x, void *d_out,
                     int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                     float *elapsed_ms, void *stream_, const uint32_t *d_luts = nullptr, int rows_per_codebook = 0,
                     int out_f32 = 0, int64_t max_tile_bytes = 0, int64_t max_stream_bytes = 0, int max_code_bits = 0,
                     const KvcFusedExtra *extra = nullptr)
{
    hipStream_t stream = (hipStream_t)stream_;
    if (tokens == 0) {
        if (elapsed_ms) *elapsed_ms = 0.f;
        return 0;
    }
    KVC_REQUIRE(batch > 0 && kv_heads > 0 && q_heads > 0 && q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads");
    const int64_t rep = q_heads / kv_heads;
    KVC_REQUIRE(rep == 1 || rep == 2 || rep == 4 || rep == 8, "q_heads / kv_heads must be 1, 2, 4 or 8");
    if (is_k) {
        KVC_REQUIRE(quant_mask == KVC_MASK_K_BLOCK || quant_mask == KVC_MASK_CHANNEL,
                    "fused K supports block (0xF) and per-channel (0x1) quantization groups");
    } else {
        KVC_REQUIRE(quant_mask == KVC_MASK_V_TOKEN || quant_mask == KVC_MASK_SIM_TOKEN || quant_mask == KVC_MASK_VECTOR,
                    "fused V supports per-token quantization groups (0xE, 0xC, 0x8)");
    }
    KVC_REQUIRE(((uintptr_t)d_scale & 3) == 0 && ((uintptr_t)d_min & 1) == 0,
                "quant_scales must be 4-byte aligned and quant_min_ints 2-byte aligned");
    void *slot = nullptr;
    if (!d_luts) {
        if (int rc = kvc_workspace_slot(&slot, stream_)) return rc;
    }
    KvcFusedArgs a;
    int64_t rows;
    const int64_t stride = batch * kv_heads * head_dim;
    if (int rc = kvc_fill_stream_args(a.s, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                                      thread_infos_bytes, d_luts ? d_luts : (const uint32_t *)slot, is_k, tokens, stride,
                                      head_dim, &rows))
        return rc;
    a.s.rows_per_codebook = d_luts ? rows_per_codebook : 0;
    a.min_i8 = d_min;
    a.scale = reinterpret_cast<const __half *>(d_scale);
    a.quant_mask = quant_mask;
    a.x = reinterpret_cast<const __half *>(d_x);
    a.out = d_out;
    a.out_f32 = out_f32;
    a.out_stride = (extra && extra->out_stride) ? extra->out_stride : tokens;
    a.scores = extra ? extra->scores : nullptr;
    a.scores_stride = extra ? extra->scores_stride : 0;
    a.sm_scale = extra ? extra->sm_scale : 1.f;
    a.ml = extra ? extra->ml : nullptr;
    a.tokens = tokens;
    a.batch = (int)batch;
    a.kv_heads = (int)kv_heads;
    a.q_heads = (int)q_heads;
    a.head_dim = (int)head_dim;
    const int slots = (!is_k && head_dim % KVC_WAVE != 0) ? 2 : 1;
    const int kind = is_k ? 0 : (a.scores ? 2 : 0) + slots;
    const int rounded = kvc_option(KVC_OPT_FUSED_ROUNDED) != 0;
    // The matrix-core kernels take the common case: a codebook known to have codes of at most 7 bits, the plain or
    // skewed packed payload, results that can be stored four at a time.
    const int64_t out_stride = (extra && extra->out_stride) ? extra->out_stride : tokens;
    const int want_mfma = kvc_option(KVC_OPT_FUSED_MFMA);
    const bool mfma = want_mfma != 0 && max_code_bits >= 1 && max_code_bits <= 7 &&
                      kvc_option(KVC_OPT_FUSED_ROWS) != 1 && ((uintptr_t)d_out & 15) == 0 &&
                      (is_k ? out_stride % 4 == 0 : head_dim % 4 == 0);
    const size_t lds = mfma ? kvc_plan_lds(a, slots, (int)rep, encoded_bytes, rows * a.s.cols, max_tile_bytes, max_stream_bytes,
                                           max_code_bits, 0, true, kvc_mfma_ops_words(slots, (int)rep, rounded))
                            : kvc_plan_lds(a, slots, rounded ? (int)rep + 1 : (int)rep, encoded_bytes, rows * a.s.cols,
                                           max_tile_bytes, max_stream_bytes, max_code_bits, 0, !rounded);
    a.rounded = rounded;
    // V tiles after which the heads repeat (the kernels that keep a head's operand tables from tile to tile)
    int unit = 0;
    if (!is_k && mfma && rounded) {
        int64_t l = head_dim;
        while (l % KVC_WAVE != 0) l += head_dim;               // least common multiple of head_dim and 64
        unit = (int)(l / KVC_WAVE);
    }
    a.s.tiles_per_wave = kvc_plan_tiles_per_wave(rows * a.s.cols, unit, (int)rep);
    KvcTimer timer(elapsed_ms, stream);
    if (!d_luts) {
        if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    }
    dim3 grid = kvc_grid(a.s, rows);
    a.sched_nseg = 0;
    if (mfma) {
        if (const unsigned wgs = kvc_plan_schedule(a, rows * a.s.cols, unit, (int)rep)) grid = dim3(wgs, 1);
    }
    static const bool trace_plan = getenv("KVCOMP_TRACE_PLAN") != nullptr;
    if (trace_plan && a.sched_nseg)
        fprintf(stderr, "[kvcomp] schedule: %d segments, runs %d %d %d %d from workgroups %d %d %d %d (tiles %d %d %d %d), %d tiles\n",
                a.sched_nseg, a.sched_run[0], a.sched_run[1], a.sched_run[2], a.sched_run[3], a.sched_wg[0], a.sched_wg[1],
                a.sched_wg[2], a.sched_wg[3], a.sched_tile[0], a.sched_tile[1], a.sched_tile[2], a.sched_tile[3], a.sched_tile[4]);
    if (trace_plan)
        fprintf(stderr, "[kvcomp] fused kind %d rep %d: grid %u x %u, lds %zu B (table %d w, payload %d w of %d logical, "
                "skew %d, rows %d), pair bits %d, tiles per wave %d, rounded %d\n", kind, (int)rep, grid.x, grid.y, lds,
                a.table_words, a.pack_words, a.pack_logical, a.skew, a.row_words, a.pair_bits, a.s.tiles_per_wave, a.rounded);
    if (mfma) {
        if (trace_plan) fprintf(stderr, "[kvcomp]   matrix-core kernel\n");
        kvc_launch_fused_mfma((int)rep, kind, rounded != 0, a, grid, lds, stream);
        KVC_HIP(hipGetLastError());
        return timer.finish();
    }
    switch (rep) {
        case 1: kvc_launch_fused<1>(kind, a, grid, lds, stream); break;
        case 2: kvc_launch_fused<2>(kind, a, grid, lds, stream); break;
        case 4: kvc_launch_fused<4>(kind, a, grid, lds, stream); break;
        default: kvc_launch_fused<8>(kind, a, grid, lds, stream); break;
    }
    KVC_HIP(hipGetLastError());
    return timer.finish();
}

// Plain decode (d_out uint8 [tokens, stride]) or decode + dequantize (d_out fp16, same shape) of a whole stream.
// Returns 1 when the layout is not one the kernel handles (the caller then uses the two-step kernels).
int kvc_expand(int is_k, int deq, const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
               const uint8_t *d_block_infos, int64_t block_infos_bytes, const uint8_t *d_thread_infos,
               int64_t thread_infos_bytes, const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_min,
               const void *d_scale, int quant_mask, void *d_out, int64_t tokens, int64_t batch, int64_t heads,
               int64_t head_dim, float *elapsed_ms, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    if (head_dim <= 0 || head_dim > KVC_K_VEC_LEN || head_dim % 8 != 0) return 1;
    if (deq) {
        if (is_k && quant_mask != KVC_MASK_K_BLOCK && quant_mask != KVC_MASK_CHANNEL) return 1;
        if (!is_k && quant_mask != KVC_MASK_V_TOKEN && quant_mask != KVC_MASK_SIM_TOKEN && quant_mask != KVC_MASK_VECTOR) return 1;
    }
    KVC_REQUIRE(!deq || (((uintptr_t)d_scale & 3) == 0 && ((uintptr_t)d_min & 1) == 0),
                "quant_scales must be 4-byte aligned and quant_min_ints 2-byte aligned");
    void *slot = nullptr;
    if (int rc = kvc_workspace_slot(&slot, stream_)) return rc;
    KvcFusedArgs a;
    a.sched_nseg = 0;
    int64_t rows;
    const int64_t stride = batch * heads * head_dim;
    if (int rc = kvc_fill_stream_args(a.s, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                                      thread_infos_bytes, (const uint32_t *)slot, is_k, tokens, stride, head_dim, &rows))
        return rc;
    KVC_REQUIRE(((uintptr_t)d_out & 15) == 0, "output pointer must be 16-byte aligned");
    a.min_i8 = d_min;
    a.scale = reinterpret_cast<const __half *>(d_scale);
    a.quant_mask = deq ? quant_mask : (is_k ? KVC_MASK_K_BLOCK : KVC_MASK_V_TOKEN);
    a.x = nullptr;
    a.out = d_out;
    a.out_f32 = 0;
    a.out_stride = 0;
    a.scores = nullptr;
    a.scores_stride = 0;
    a.sm_scale = 1.f;
    a.ml = nullptr;
    a.tokens = tokens;
    a.batch = (int)batch;
    a.kv_heads = (int)heads;
    a.q_heads = (int)heads;
    a.head_dim = (int)head_dim;
    const int slots = (!is_k && head_dim % KVC_WAVE != 0) ? 2 : 1;
    const int out_words = is_k ? (deq ? KvcSlab<true, true>::WORDS : KvcSlab<true, false>::WORDS)
                               : (deq ? KvcSlab<false, true>::WORDS : KvcSlab<false, false>::WORDS);
    const size_t lds = kvc_plan_lds(a, slots, deq ? 1 : 0, encoded_bytes, rows * a.s.cols, 0, 0, 0, out_words);
    a.expand = deq ? 2 : 1;
    a.out_words = out_words;
    // One tile per wave: measured on MI355X at 65 536 K / 49 152 V tiles, plain decode runs 1.2 to 1.4 times faster
    // than with two (K symbols 1.6 -> 2.3 TB/s out), decode + dequantize 1.05 to 1.1 times: nothing here is built once
    // per wave that a second tile could share, and shorter waves balance better over the chip.
    const int forced_tpw = kvc_option(KVC_OPT_FUSED_TILES_PER_WAVE);
    a.s.tiles_per_wave = forced_tpw > 0 ? (forced_tpw > 64 ? 64 : forced_tpw) : 1;
    KvcTimer timer(elapsed_ms, stream);
    if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    const dim3 grid = kvc_grid(a.s, rows);
    const int kind = is_k ? 0 : slots;
#define KVC_EXPAND_LAUNCH(K, Q) hipLaunchKernelGGL((kvc_expand_kernel<K, Q>), grid, dim3(KVC_WG), lds, stream, a)
    if (deq) {
        if (kind == 0) KVC_EXPAND_LAUNCH(0, true);
        else if (kind == 1) KVC_EXPAND_LAUNCH(1, true);
        else KVC_EXPAND_LAUNCH(2, true);
    } else {
        if (kind == 0) KVC_EXPAND_LAUNCH(0, false);
        else if (kind == 1) KVC_EXPAND_LAUNCH(1, false);
        else KVC_EXPAND_LAUNCH(2, false);
    }
#undef KVC_EXPAND_LAUNCH
    KVC_HIP(hipGetLastError());
    return timer.finish();
}

extern "C" int kvc_k_decode_and_mat_vec_mul(const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                            const uint8_t *d_block_infos, int64_t block_infos_bytes,
                                            const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                            const uint8_t *d_encoded, int64_t encoded_bytes,
                                            const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                                            const void *d_q_f16, void *d_scores_f16, int64_t tokens, int64_t batch,
                                            int64_t kv_heads, int64_t q_heads, int64_t head_dim, float *elapsed_ms,
                                            void *stream)
{
    return kvc_fused(1, d_decode_tree, decode_tree_bytes, tree_format, d_block_infos, block_infos_bytes, d_thread_infos,
                     thread_infos_bytes, d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask,
                     d_q_f16, d_scores_f16, tokens, batch, kv_heads, q_heads, head_dim, elapsed_ms, stream);
}

extern "C" int kvc_v_decode_and_mat_vec_mul(const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                            const uint8_t *d_block_infos, int64_t block_infos_bytes,
                                            const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                            const uint8_t *d_encoded, int64_t encoded_bytes,
                                            const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                                            const void *d_p_f16, void *d_partial_f16, int64_t tokens, int64_t batch,
                                            int64_t kv_heads, int64_t q_heads, int64_t head_dim, float *elapsed_ms,
                                            void *stream)
{
    return kvc_fused(0, d_decode_tree, decode_tree_bytes, tree_format, d_block_infos, block_infos_bytes, d_thread_infos,
                     thread_infos_bytes, d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask,
                     d_p_f16, d_partial_f16, tokens, batch, kv_heads, q_heads, head_dim, elapsed_ms, stream);
}

// ---------------------------------------------------------------------------------------------------
// variants that take decode tables built once with kvc_build_lut (no per-call table construction)
// ---------------------------------------------------------------------------------------------------
extern "C" int64_t kvc_lut_bytes(void) { return KVC_LUT_BYTES; }

extern "C" int kvc_build_lut(const uint8_t *d_decode_trees, int64_t tree_bytes, int tree_format, int64_t n_codebooks,
                             int64_t tree_stride_bytes, void *d_luts, void *stream)
{
    KVC_REQUIRE(n_codebooks >= 1 && n_codebooks <= 65535, "bad codebook count");
    KVC_REQUIRE(((uintptr_t)d_luts & 15) == 0, "table buffer must be 16-byte aligned");
    return kvc_launch_build_lut(d_decode_trees, tree_bytes, tree_format, (uint32_t *)d_luts, (int)n_codebooks,
                                tree_stride_bytes, (hipStream_t)stream);
}

extern "C" int kvc_k_scores_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                                int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                                const void *d_quant_scales_f16, int quant_mask, const void *d_q_f16, void *d_scores,
                                int out_f32, int64_t max_tile_bytes, int64_t max_stream_bytes, int max_code_bits, int64_t tokens, int64_t batch, int64_t kv_heads,
                                int64_t q_heads, int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(1, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_q_f16, d_scores, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32, max_tile_bytes, max_stream_bytes, max_code_bits);
}

extern "C" int kvc_v_partials_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                                  int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                  const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                                  const void *d_quant_scales_f16, int quant_mask, const void *d_p_f16, void *d_partial,
                                  int out_f32, int64_t max_tile_bytes, int64_t max_stream_bytes, int max_code_bits, int64_t tokens, int64_t batch, int64_t kv_heads,
                                  int64_t q_heads, int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(0, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_p_f16, d_partial, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32, max_tile_bytes, max_stream_bytes, max_code_bits);
}

// ---------------------------------------------------------------------------------------------------
// one-call decode attention over a compressed cache (no counterpart in the reference, whose models
// decompress everything and run dense attention; models/cache/kvcomp_quant.py:74-75)
//
//   scores  = q . K^T        compressed part: fused K kernel; fp16 tail: kvc_tail_scores_kernel
//   groups  of 128 tokens    compressed part: fused V kernel in softmax mode -> (m_g, l_g, sum_t w_t v_t);
//                            fp16 tail: kvc_tail_values_kernel -> one more group
//   out     = sum_g e^(m_g - M) part_g / sum_g e^(m_g - M) l_g          kvc_attention_combine_kernel
//
// Every 128-token group carries its own running maximum, so no pass over all scores is needed before the
// values are read (the split-softmax scheme of flash decoding).
// ---------------------------------------------------------------------------------------------------

// scores[b, hq, t0 + t] = sum_d tail[t, b, h, d] q[b, hq, d]; one wave per (t, b, h), lanes over d
__global__ void __launch_bounds__(KVC_WG)
kvc_tail_scores_kernel(const __half *__restrict__ tail, const __half *__restrict__ q, float *__restrict__ scores,
                       int64_t scores_stride, int64_t t0, int64_t tail_tokens, int batch, int kv_heads, int rep, int D)
{
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + (threadIdx.x >> 6);
    if (item >= tail_tokens * batch * kv_heads) return;
    const int h = (int)(item % kv_heads);
    const int b = (int)((item / kv_heads) % batch);
    const int64_t t = item / ((int64_t)kv_heads * batch);
    const __half *kp = tail + item * D;
    float k0 = 0.f, k1 = 0.f;
    if (2 * lane < D) {
        const __half2 v = *reinterpret_cast<const __half2 *>(kp + 2 * lane);
        k0 = __low2float(v);
        k1 = __high2float(v);
    }
    for (int r = 0; r < rep; r++) {
        const int hq = h * rep + r;
        const __half *qp = q + ((int64_t)b * kv_heads * rep + hq) * D;
        float acc = 0.f;
        if (2 * lane < D) {
            const __half2 v = *reinterpret_cast<const __half2 *>(qp + 2 * lane);
            acc = k0 * __low2float(v) + k1 * __high2float(v);
        }
        acc = kvc_wave_sum_dpp(acc);
        if (lane == 0) scores[((int64_t)b * kv_heads * rep + hq) * scores_stride + t0 + t] = acc;
    }
}

// The tail tokens [t0, t0 + n) as one more group: one workgroup of four waves per (b, hq).  The tokens are taken
// 256 at a time: every thread turns one score into a weight (against the group's maximum, found first), then wave w
// adds tokens w, w + 4, ... of the chunk, lane l holding channels 2l and 2l + 1 (one coalesced row read per token).
constexpr int KVC_TAIL_WAVES = 4;
__global__ void __launch_bounds__(KVC_TAIL_WAVES * KVC_WAVE)
kvc_tail_values_kernel(const __half *__restrict__ tail, const float *__restrict__ scores, int64_t scores_stride,
                       float sm_scale, float *__restrict__ part, float *__restrict__ ml, int64_t t0, int64_t n,
                       int batch, int kv_heads, int rep, int D)
{
    constexpr int CHUNK = KVC_TAIL_WAVES * KVC_WAVE;
    __shared__ float s_red[KVC_TAIL_WAVES];
    __shared__ float s_w[CHUNK];
    __shared__ float s_acc[KVC_TAIL_WAVES][2 * KVC_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hq = blockIdx.x % (kv_heads * rep), b = blockIdx.x / (kv_heads * rep);
    const int h = hq / rep;
    const float *sp = scores + ((int64_t)b * kv_heads * rep + hq) * scores_stride + t0;
    // the group's maximum
    float m = -INFINITY;
    for (int64_t t = tid; t < n; t += CHUNK) m = fmaxf(m, sp[t] * sm_scale);
    m = kvc_wave_fmax_dpp(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = s_red[0];
#pragma unroll
    for (int w = 1; w < KVC_TAIL_WAVES; w++) m = fmaxf(m, s_red[w]);
    float l = 0.f, acc0 = 0.f, acc1 = 0.f;
    const bool live = 2 * lane < D;
    const int64_t row = (int64_t)batch * kv_heads * D;                  // halves per token
    const __half *vp = tail + ((int64_t)b * kv_heads + h) * D + (live ? 2 * lane : 0);
    for (int64_t c0 = 0; c0 < n; c0 += CHUNK) {
        const int64_t t = c0 + tid;
        const float w = t < n ? __expf(sp[t] * sm_scale - m) : 0.f;
        __syncthreads();                                               // the previous chunk's weights have been used
        s_w[tid] = w;
        l += w;
        __syncthreads();
        const int len = (int)(n - c0 < CHUNK ? n - c0 : CHUNK);
        for (int k = wave; k < len; k += KVC_TAIL_WAVES) {
            const float wk = s_w[k];
            const __half2 v = *reinterpret_cast<const __half2 *>(vp + (c0 + k) * row);
            acc0 += wk * __low2float(v);
            acc1 += wk * __high2float(v);
        }
    }
    l = kvc_wave_sum_dpp(l);
    __syncthreads();
    if (lane == 0) s_red[wave] = l;
    s_acc[wave][2 * lane] = acc0;
    s_acc[wave][2 * lane + 1] = acc1;
    __syncthreads();
    if (tid < D) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < KVC_TAIL_WAVES; w++) a += s_acc[w][tid];
        part[((int64_t)b * kv_heads * rep + hq) * D + tid] = a;
    }
    if (tid == 0) {
        float lsum = 0.f;
#pragma unroll
        for (int w = 0; w < KVC_TAIL_WAVES; w++) lsum += s_red[w];
        ml[((int64_t)b * kv_heads * rep + hq) * 2] = m;
        ml[((int64_t)b * kv_heads * rep + hq) * 2 + 1] = lsum;
    }
}

// out[b, hq, :] from `groups` partials; one workgroup of 16 waves per (b, hq), wave w takes groups w, w + 16, ...
// Each wave sums its groups relative to a maximum of its own -- U groups at a time, all their loads issued
// together (indices past the end are clamped and weighted zero, so nothing branches around a load) -- and the
// waves' sums are brought to the common maximum when they are merged: a 32k-token context is one round trip to
// memory and one barrier.
// With tail.n_v > 0 the same workgroup first handles the tokens that V keeps uncompressed (at most
// KVC_FINISH_MAX_TAIL), as one more group: their scores (from the score matrix where K had them compressed, else
// q . the fp16 row of K's tail), the group's maximum, the weights and the weighted sum of V's fp16 rows.
constexpr int KVC_COMBINE_WAVES = 16;
constexpr int KVC_FINISH_MAX_TAIL = KVC_COMBINE_WAVES * KVC_WAVE;
struct KvcTailArgs {
    const __half *k_tail, *v_tail, *q;    // [n_k, B, H, D], [n_v, B, H, D], [B, Hq, D]
    const float *scores;                  // [B * Hq, scores_stride], filled for tokens below kc
    int64_t scores_stride;
    int64_t kc, vc;                       // tokens that K / V hold compressed (kc >= vc)
    int n_k, n_v;                         // tokens in K's / V's fp16 tail (total - kc, total - vc)
    float sm_scale;
    int batch, kv_heads, rep;
};

template <int U>
__global__ void __launch_bounds__(KVC_COMBINE_WAVES * KVC_WAVE)
kvc_attention_combine_kernel(const float *__restrict__ part, const float *__restrict__ ml, int64_t groups,
                             int64_t bhq_count, int D, float *__restrict__ out, KvcTailArgs tail)
{
    __shared__ float s_max[KVC_COMBINE_WAVES];
    __shared__ float s_num[KVC_COMBINE_WAVES][128];
    __shared__ float s_den[KVC_COMBINE_WAVES];
    __shared__ float s_w[KVC_FINISH_MAX_TAIL];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t bhq = blockIdx.x;
    const int d0 = lane < D ? lane : 0, d1 = lane + 64 < D ? lane + 64 : 0;
    float M = -INFINITY, n0 = 0.f, n1 = 0.f, den = 0.f;   // this wave's running maximum and its sums relative to it
    for (int64_t g0 = wave; g0 < groups; g0 += U * KVC_COMBINE_WAVES) {
        float mg[U], lg[U], p0[U], p1[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int64_t g = g0 + u * KVC_COMBINE_WAVES;
            const int64_t gc = g < groups ? g : groups - 1;
            const float *mlp = ml + (gc * bhq_count + bhq) * 2;
            const float *pp = part + (gc * bhq_count + bhq) * D;
            mg[u] = g < groups ? mlp[0] : -INFINITY;
            lg[u] = mlp[1];
            p0[u] = pp[d0];
            p1[u] = pp[d1];
        }
        float mb = mg[0];
#pragma unroll
        for (int u = 1; u < U; u++) mb = fmaxf(mb, mg[u]);
        if (mb > M) {                                     // wave-uniform; rescale what has been summed so far
            const float f = __expf(M - mb);               // exp(-inf) = 0 the first time
            n0 *= f;
            n1 *= f;
            den *= f;
            M = mb;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float f = __expf(mg[u] - M);            // 0 for the slots past the end (M is finite here)
            den += f * lg[u];
            n0 += f * p0[u];
            n1 += f * p1[u];
        }
    }
    if (tail.n_v > 0) {                                   // uniform over the workgroup
        const int hq = (int)(bhq % (tail.kv_heads * tail.rep)), b = (int)(bhq / (tail.kv_heads * tail.rep));
        const int h = hq / tail.rep;
        const int from_k = (int)(tail.kc - tail.vc);      // tail tokens of V whose scores the K kernel wrote
        // scaled scores of the tail tokens
        if (tid < from_k) s_w[tid] = tail.scores[bhq * tail.scores_stride + tail.vc + tid] * tail.sm_scale;
        {
            const bool live = 2 * lane < D;
            const int e = live ? 2 * lane : 0;
            const __half2 qv = *reinterpret_cast<const __half2 *>(tail.q + bhq * D + e);
            const float q0 = live ? __low2float(qv) : 0.f, q1 = live ? __high2float(qv) : 0.f;
            const int64_t row = (int64_t)tail.batch * tail.kv_heads * D;
            const __half *kp = tail.k_tail + ((int64_t)b * tail.kv_heads + h) * D + e;
            for (int j = wave; j < tail.n_k; j += KVC_COMBINE_WAVES) {
                const __half2 kv = *reinterpret_cast<const __half2 *>(kp + j * row);
                const float dot = kvc_wave_sum_dpp(q0 * __low2float(kv) + q1 * __high2float(kv));
                if (lane == 0) s_w[from_k + j] = dot * tail.sm_scale;
            }
        }
        __syncthreads();
        // the group's maximum, then every thread turns one score into a weight
        const float sc = tid < tail.n_v ? s_w[tid] : -INFINITY;
        float mt = kvc_wave_fmax_dpp(sc);
        if (lane == 0) s_max[wave] = mt;
        __syncthreads();
        mt = s_max[0];
#pragma unroll
        for (int w = 1; w < KVC_COMBINE_WAVES; w++) mt = fmaxf(mt, s_max[w]);
        const float wt = tid < tail.n_v ? __expf(sc - mt) : 0.f;
        __syncthreads();                                  // every thread has read s_max and its score
        s_w[tid] = wt;
        const float lw = kvc_wave_sum_dpp(wt);            // this wave's share of the group's sum of weights
        __syncthreads();
        // weighted rows of V's tail: wave w takes tokens w, w + 16, ...; lane l channels l and l + 64
        float a0 = 0.f, a1 = 0.f;
        {
            const int64_t row = (int64_t)tail.batch * tail.kv_heads * D;
            const __half *vp = tail.v_tail + ((int64_t)b * tail.kv_heads + h) * D;
            for (int j = wave; j < tail.n_v; j += KVC_COMBINE_WAVES) {
                const float wj = s_w[j];
                a0 += wj * __half2float(vp[j * row + d0]);
                a1 += wj * __half2float(vp[j * row + d1]);
            }
        }
        if (mt > M) {
            const float f = __expf(M - mt);
            n0 *= f;
            n1 *= f;
            den *= f;
            M = mt;
        }
        const float f = __expf(mt - M);
        den += f * lw;
        n0 += f * a0;
        n1 += f * a1;
        __syncthreads();                                  // s_max is reused below
    }
    if (lane == 0) s_max[wave] = M;
    __syncthreads();
    float Mall = s_max[0];
#pragma unroll
    for (int w = 1; w < KVC_COMBINE_WAVES; w++) Mall = fmaxf(Mall, s_max[w]);
    const float fw = M == -INFINITY ? 0.f : __expf(M - Mall);          // a wave without groups contributes nothing
    s_num[wave][lane] = lane < D ? n0 * fw : 0.f;
    s_num[wave][lane + 64] = lane + 64 < D ? n1 * fw : 0.f;
    if (lane == 0) s_den[wave] = den * fw;
    __syncthreads();
    if (threadIdx.x < D) {
        const int d = threadIdx.x;
        float num = 0.f, dn = 0.f;
#pragma unroll
        for (int w = 0; w < KVC_COMBINE_WAVES; w++) {
            num += s_num[w][d];
            dn += s_den[w];
        }
        out[bhq * D + d] = num / dn;
    }
}

static int64_t kvc_round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

struct KvcAttentionPlan {
    int64_t total_tokens, scores_stride, groups;
    int64_t scores_off, part_off, ml_off, bytes;
};

static KvcAttentionPlan kvc_attention_plan(int64_t total_tokens, int64_t v_compressed_tokens, int64_t batch, int64_t q_heads,
                                           int64_t head_dim)
{
    KvcAttentionPlan p;
    p.total_tokens = total_tokens;
    p.scores_stride = kvc_round_up(total_tokens, 4);
    p.groups = v_compressed_tokens / KVC_V_TOKENS + (total_tokens > v_compressed_tokens ? 1 : 0);
    p.scores_off = 0;
    p.part_off = kvc_round_up(batch * q_heads * p.scores_stride * 4, 256);
    p.ml_off = p.part_off + kvc_round_up(p.groups * batch * q_heads * head_dim * 4, 256);
    p.bytes = p.ml_off + kvc_round_up(p.groups * batch * q_heads * 2 * 4, 256);
    return p;
}

extern "C" int64_t kvc_attention_workspace_bytes(int64_t total_tokens, int64_t v_compressed_tokens, int64_t batch,
                                                 int64_t q_heads, int64_t head_dim)
{
    if (total_tokens <= 0 || v_compressed_tokens < 0 || batch <= 0 || q_heads <= 0 || head_dim <= 0) return 0;
    return kvc_attention_plan(total_tokens, v_compressed_tokens, batch, q_heads, head_dim).bytes;
}

static int kvc_attention_run(const kvc_compressed_desc *k, const kvc_compressed_desc *v, const void *d_q_f16,
                             float softmax_scale, void *d_workspace, int64_t workspace_bytes, float *d_out_f32,
                             int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                             float *elapsed_ms, float *fused_kernel_ms, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    if (fused_kernel_ms) fused_kernel_ms[0] = fused_kernel_ms[1] = 0.f;
    KVC_REQUIRE(k != nullptr && v != nullptr && d_q_f16 != nullptr && d_out_f32 != nullptr, "NULL argument");
    KVC_REQUIRE(batch > 0 && kv_heads > 0 && q_heads > 0 && q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads");
    KVC_REQUIRE(head_dim > 0 && head_dim <= 128 && head_dim % 8 == 0, "head_dim must be a multiple of 8, <= 128");
    const int64_t total = k->tokens + k->tail_tokens;
    KVC_REQUIRE(total > 0, "the cache is empty");
    KVC_REQUIRE(v->tokens + v->tail_tokens == total, "K holds %lld tokens, V %lld", (long long)total,
                (long long)(v->tokens + v->tail_tokens));
    KVC_REQUIRE(k->tokens % KVC_K_VEC_PER_BLK == 0 && v->tokens % KVC_V_VEC_LEN == 0, "compressed token counts must be whole tiles");
    KVC_REQUIRE((k->tokens == 0 || k->d_luts) && (v->tokens == 0 || v->d_luts), "decode tables are required");
    KVC_REQUIRE((k->tail_tokens == 0 || k->d_tail_f16) && (v->tail_tokens == 0 || v->d_tail_f16), "tail pointer is NULL");
    const KvcAttentionPlan p = kvc_attention_plan(total, v->tokens, batch, q_heads, head_dim);
    KVC_REQUIRE(d_workspace != nullptr && ((uintptr_t)d_workspace & 255) == 0, "workspace must be 256-byte aligned");
    KVC_REQUIRE(workspace_bytes >= p.bytes, "workspace holds %lld bytes, %lld needed", (long long)workspace_bytes, (long long)p.bytes);
    float *scores = reinterpret_cast<float *>((char *)d_workspace + p.scores_off);
    float *part = reinterpret_cast<float *>((char *)d_workspace + p.part_off);
    float *ml = reinterpret_cast<float *>((char *)d_workspace + p.ml_off);
    const int rep = (int)(q_heads / kv_heads);
    KvcTimer timer(elapsed_ms, stream);
    // ---- scores
    if (k->tokens) {
        KvcFusedExtra ex = {p.scores_stride, nullptr, 0, 1.f, nullptr};
        if (int rc = kvc_fused(1, nullptr, 0, KVC_TREE_I8, k->d_block_infos, k->block_infos_bytes, k->d_thread_infos,
                               k->thread_infos_bytes, k->d_encoded, k->encoded_bytes, k->d_quant_min_ints,
                               k->d_quant_scales_f16, k->quant_mask, d_q_f16, scores, k->tokens, batch, kv_heads, q_heads,
                               head_dim, fused_kernel_ms, stream_, (const uint32_t *)k->d_luts, (int)k->rows_per_codebook, 1,
                               k->max_tile_bytes, k->max_stream_bytes, k->max_code_bits, &ex))
            return rc;
    }
    // V's fp16 tail is handled by the merge kernel itself when it is short enough and K's compressed part reaches at
    // least as far as V's (the V kernel then needs no score of K's tail); otherwise by two kernels of its own
    KvcTailArgs tail = {};
    const bool tail_in_merge = v->tail_tokens > 0 && v->tail_tokens <= KVC_FINISH_MAX_TAIL && k->tokens >= v->tokens &&
                               kvc_option(KVC_OPT_ATTENTION_TAIL_IN_MERGE) != 0;
    if (tail_in_merge) {
        tail.k_tail = reinterpret_cast<const __half *>(k->d_tail_f16);
        tail.v_tail = reinterpret_cast<const __half *>(v->d_tail_f16);
        tail.q = reinterpret_cast<const __half *>(d_q_f16);
        tail.scores = scores;
        tail.scores_stride = p.scores_stride;
        tail.kc = k->tokens;
        tail.vc = v->tokens;
        tail.n_k = (int)k->tail_tokens;
        tail.n_v = (int)v->tail_tokens;
        tail.sm_scale = softmax_scale;
        tail.batch = (int)batch;
        tail.kv_heads = (int)kv_heads;
        tail.rep = rep;
    }
    if (k->tail_tokens && !tail_in_merge) {
        const int64_t items = k->tail_tokens * batch * kv_heads;
        hipLaunchKernelGGL(kvc_tail_scores_kernel, dim3((unsigned)((items + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG)), dim3(KVC_WG),
                           0, stream, reinterpret_cast<const __half *>(k->d_tail_f16), reinterpret_cast<const __half *>(d_q_f16),
                           scores, p.scores_stride, k->tokens, k->tail_tokens, (int)batch, (int)kv_heads, rep, (int)head_dim);
    }
    // ---- weighted values per group
    if (v->tokens) {
        KvcFusedExtra ex = {0, scores, p.scores_stride, softmax_scale, ml};
        if (int rc = kvc_fused(0, nullptr, 0, KVC_TREE_I8, v->d_block_infos, v->block_infos_bytes, v->d_thread_infos,
                               v->thread_infos_bytes, v->d_encoded, v->encoded_bytes, v->d_quant_min_ints,
                               v->d_quant_scales_f16, v->quant_mask, nullptr, part, v->tokens, batch, kv_heads, q_heads,
                               head_dim, fused_kernel_ms ? fused_kernel_ms + 1 : nullptr, stream_, (const uint32_t *)v->d_luts, (int)v->rows_per_codebook, 1,
                               v->max_tile_bytes, v->max_stream_bytes, v->max_code_bits, &ex))
            return rc;
    }
    if (v->tail_tokens && !tail_in_merge) {
        const int64_t g = v->tokens / KVC_V_TOKENS;
        hipLaunchKernelGGL(kvc_tail_values_kernel, dim3((unsigned)(batch * q_heads)), dim3(KVC_TAIL_WAVES * KVC_WAVE), 0, stream,
                           reinterpret_cast<const __half *>(v->d_tail_f16), scores, p.scores_stride, softmax_scale,
                           part + g * batch * q_heads * head_dim, ml + g * batch * q_heads * 2, v->tokens, v->tail_tokens,
                           (int)batch, (int)kv_heads, rep, (int)head_dim);
    }
    // groups in flight per wave: what one pass over a wave's share needs, at most 16
    const int64_t groups = tail_in_merge ? v->tokens / KVC_V_TOKENS : p.groups;
    const dim3 cgrid((unsigned)(batch * q_heads)), cblock(KVC_COMBINE_WAVES * KVC_WAVE);
    const int64_t per_wave = (groups + KVC_COMBINE_WAVES - 1) / KVC_COMBINE_WAVES;
    if (per_wave <= 4)
        hipLaunchKernelGGL(kvc_attention_combine_kernel<4>, cgrid, cblock, 0, stream, part, ml, groups, batch * q_heads, (int)head_dim, d_out_f32, tail);
    else if (per_wave <= 8)
        hipLaunchKernelGGL(kvc_attention_combine_kernel<8>, cgrid, cblock, 0, stream, part, ml, groups, batch * q_heads, (int)head_dim, d_out_f32, tail);
    else
        hipLaunchKernelGGL(kvc_attention_combine_kernel<16>, cgrid, cblock, 0, stream, part, ml, groups, batch * q_heads, (int)head_dim, d_out_f32, tail);
    KVC_HIP(hipGetLastError());
    return timer.finish();
}

extern "C" int kvc_attention_decode(const kvc_compressed_desc *k, const kvc_compressed_desc *v, const void *d_q_f16,
                                    float softmax_scale, void *d_workspace, int64_t workspace_bytes, float *d_out_f32,
                                    int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                                    float *elapsed_ms, float *fused_kernel_ms, void *stream_)
{
    return kvc_attention_run(k, v, d_q_f16, softmax_scale, d_workspace, workspace_bytes, d_out_f32, batch, kv_heads,
                             q_heads, head_dim, elapsed_ms, fused_kernel_ms, stream_);
}

// ---------------------------------------------------------------------------------------------------
// The same operator for callers that may not allocate (code under HIP graph capture, serving loops with a
// fixed memory plan): the workspace (scores, per-group partials and their (max, sum) pairs) lives in a
// device array of this library instead of a caller's buffer.  Every device holds its own copy of the
// array at its own address; the address is looked up once per device, on the first call there, and only
// that pointer -- never the array's name, which in host code is a stand-in and not a device address --
// is handed to the kernels.  Nothing in the workspace has to start at zero: every word the kernels read
// is written earlier in the same call (scores by the K kernel, partials and (max, sum) by the V kernel),
// at offsets that depend on this call's shape alone, so what an earlier, larger call left behind is
// never read.  Calls that overlap in time on one device share the array and race.
// ---------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[KVC_ATTENTION_STATIC_SCRATCH_BYTES];
constexpr int KVC_SCRATCH_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[KVC_SCRATCH_MAX_DEVICES] = {};

static int kvc_static_scratch(void **ptr)
{
    int dev = 0;
    KVC_HIP(hipGetDevice(&dev));
    KVC_REQUIRE(dev >= 0 && dev < KVC_SCRATCH_MAX_DEVICES, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        KVC_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        KVC_REQUIRE(p != nullptr && ((uintptr_t)p & 255) == 0, "the static workspace has no usable device address");
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" int kvc_attention_decode_static(const kvc_compressed_desc *k, const kvc_compressed_desc *v, const void *d_q_f16,
                                           float softmax_scale, float *d_out_f32, int64_t batch, int64_t kv_heads,
                                           int64_t q_heads, int64_t head_dim, void *stream_)
{
    KVC_REQUIRE(k != nullptr && v != nullptr, "NULL argument");
    KVC_REQUIRE(batch > 0 && q_heads > 0 && head_dim > 0, "batch, q_heads and head_dim must be positive");
    const int64_t total = k->tokens + k->tail_tokens;
    KVC_REQUIRE(total > 0 && v->tokens >= 0, "the cache is empty");
    const int64_t need = kvc_attention_plan(total, v->tokens, batch, q_heads, head_dim).bytes;
    KVC_REQUIRE(need <= (int64_t)KVC_ATTENTION_STATIC_SCRATCH_BYTES,
                "this shape needs a workspace of %lld bytes, the static one holds %lld: use kvc_attention_decode",
                (long long)need, (long long)KVC_ATTENTION_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (int rc = kvc_static_scratch(&ws)) return rc;
    return kvc_attention_run(k, v, d_q_f16, softmax_scale, ws, (int64_t)KVC_ATTENTION_STATIC_SCRATCH_BYTES, d_out_f32, batch,
                             kv_heads, q_heads, head_dim, nullptr, nullptr, stream_);
}
