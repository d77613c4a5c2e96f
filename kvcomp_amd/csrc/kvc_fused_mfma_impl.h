// kvc_fused_mfma_impl.h -- the fused decode + matvec kernels with the multiply-accumulate on the matrix cores.
//
//   kvc_fused_mfma_kernel<REP, 0, ROUNDED>      <- huffman_decode_and_mat_vec_mul   (kvcomp_cuda_extension/src/kernels.cu:721-776)
//   kvc_fused_mfma_kernel<REP, 1 .. 4, ROUNDED> <- v_huffman_decode_and_mat_vec_mul (kernels.cu:778-861)
//
// Same work split, tile pipeline and lock-step table decode as kvc_fused.hip (one wave64 per tile, lane = stream, every
// lane decodes element i of its stream at step i).  What differs is where the products are formed.  A lane keeps the
// last four decoded elements as four fp16 in two registers, and one v_mfma_f32_4x4x4_16b_f16 multiplies them with the
// wave-uniform operands of those four elements: the instruction computes, for each of its 16 blocks of four lanes,
//   D[i][j] += sum_k A[i][k] B[k][j]        A[i][k]: element k of lane 4 block + i     (what the lane decoded)
//                                           B[k][j]: held by lane 4 block + j          (operand column j)
//                                           D[i][j]: register i of lane 4 block + j
// so the 64 rows are the 64 lane streams (K: tokens, V: channels), k runs over four consecutive elements (K: channels,
// V: tokens of the group) and the four columns are operand vectors.  Every query head owns two columns, the high and
// the low fp16 part of its fp32 weight (the low part scaled by 4096, so both parts stay normal numbers): symbols are
// exact in fp16, products of two fp16 are exact in the fp32 accumulator, and hi + lo / 4096 carries 22 bits of the
// weight, so the result is as accurate as the fp32 FMA loop's.  One matrix instruction replaces 4 x REP FMAs, and the
// operand comes from one 8-byte LDS read per lane (its own column: four addresses per wave).
//
// Rounded mode (KvcFusedArgs::rounded): every dequantized value is rounded to fp16 before it is multiplied, as the
// reference's dequantizer rounds it (models/cache/kvcomp_encode.py:146): two elements at a time with one packed
// fp16 add (sym + min, exact) and one packed fp16 multiply (one rounding of the exact product), the pairs of minima
// and scales of a group of four elements arriving in one 16-byte broadcast read; the columns then hold q / the
// softmax weights themselves.
//
// Tables: the one-symbol table holds {symbol as fp16, upper half; code length, lowest byte}.  Where twice the longest
// code fits KvcFusedArgs::pair_bits and every symbol's fp16 pattern has its five lowest bits clear (symbols below 64,
// and multiples of a power of two beyond), a two-symbol table {second symbol fp16 | first symbol fp16 | both lengths
// in the lowest five bits} halves the look-ups; it is four bytes per entry, so it costs half the LDS cycles of an
// eight-byte one.
//
// Everything that is not the common case (codes longer than 7 bits or than the table index, tiles that do not fit
// the staging area) is decoded one symbol at a time by kvc_mfma_slow_tile, which reads the same operand tables.
#pragma once
#include "kvc_fused_common.h"

typedef _Float16 kvc_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 kvc_h4 __attribute__((ext_vector_type(4)));
typedef float kvc_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t kvc_w2 __attribute__((ext_vector_type(2)));
typedef uint32_t kvc_w4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) kvc_w2 kvc_lds_w2;
typedef __attribute__((address_space(3))) kvc_w4 kvc_lds_w4;

constexpr float KVC_LO_SCALE = 4096.f;
constexpr uint32_t KVC_PAIR_LEN_MASK = 0x1fu;      // both code lengths of a two-symbol entry (at most 30)

__device__ __forceinline__ uint32_t kvc_lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// BCAST: every block of four lanes takes its operand columns from lanes 0 - 15 (the instruction's lane-group pattern 4),
// so only those sixteen lanes have to hold them.
template <bool BCAST>
__device__ __forceinline__ kvc_f4 kvc_mfma4(uint32_t a01, uint32_t a23, kvc_w2 b, kvc_f4 c)
{
    const kvc_w2 a = {a01, a23};
    if (BCAST) return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(kvc_h4, a), __builtin_bit_cast(kvc_h4, b), c, 0, 0, 4);
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(kvc_h4, a), __builtin_bit_cast(kvc_h4, b), c, 0, 0, 0);
}

// This lane's operand columns of one group: an 8-byte LDS read, by the first sixteen lanes only where they serve all.
template <bool BCAST>
__device__ __forceinline__ kvc_w2 kvc_read_columns(uint32_t addr, bool holder)
{
    kvc_w2 b;
    // whatever the registers hold: with the broadcast the matrix core reads the operand from the first sixteen lanes
    // and from no other, so the rest need no defined value (and no instruction to give them one)
    asm volatile("" : "=v"(b.x), "=v"(b.y));
    if (!BCAST || holder) b = *(const kvc_lds_w2 *)(uintptr_t)addr;
    return b;
}

// {x.lo, x.hi} -> RN16((x + mn) * sc) per half: the sum of two small integers is exact in fp16, the product is
// rounded once
__device__ __forceinline__ uint32_t kvc_dequant_pair(uint32_t x, uint32_t mn, uint32_t sc)
{
    const kvc_h2 v = (__builtin_bit_cast(kvc_h2, x) + __builtin_bit_cast(kvc_h2, mn)) * __builtin_bit_cast(kvc_h2, sc);
    return __builtin_bit_cast(uint32_t, v);
}

// upper halves of two table entries side by side: {a >> 16, b >> 16 << 16}
__device__ __forceinline__ uint32_t kvc_pack_hi16(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

// -- operand tables -----------------------------------------------------------------------------------
// btab  [slot][group g][set][column j][element k]  fp16: weight part of element 4 g + k for column 4 set + j;
//       column 2 r is the high part of query head r's weight, column 2 r + 1 its low part times 4096
// mstab [slot][group g] = {min 4g, min 4g+1 | min 4g+2, min 4g+3 | scale 4g, 4g+1 | scale 4g+2, 4g+3}  (rounded mode)
template <int REP>
struct KvcMfmaTables {
    static constexpr int NM = kvc_mfma_sets(REP);
    static constexpr int BTAB_SLOT_WORDS = KVC_MFMA_GROUPS * NM * 8;
    static constexpr int MSTAB_SLOT_WORDS = KVC_MFMA_GROUPS * 4;
};

__device__ __forceinline__ uint32_t kvc_half_pair(float lo, float hi)
{
    return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
}

// Split v into a high fp16 part (zero where it would be subnormal) and the remainder times 4096 as fp16.
__device__ __forceinline__ void kvc_split_weight(float v, float &hi, float &lo)
{
    const float h = __half2float(__float2half_rn(v));
    hi = fabsf(h) < 6.103515625e-5f ? 0.f : h;
    lo = (v - hi) * KVC_LO_SCALE;
}

// Rounded mode: the minima of a lane's two elements as two fp16, and their two scales, in the order the decode loops read
// them.  Where both elements' parameters came in one word each (wave-uniform `pmode`), the scales are that word and the
// two int8 minima are converted together: the byte m ^ 0x80 = m + 128 under the byte 0x64 is the fp16 number 1152 + m.
template <class Raw>
__device__ __forceinline__ void kvc_mfma_min_scale_words(const Raw &raw, int s, int pmode, uint32_t &mins, uint32_t &scales)
{
    if (pmode == KVC_PAIR_ADJACENT) {
        const uint32_t biased = __builtin_amdgcn_perm(0x64u, raw.mnw[s][0] ^ 0x8080u, 0x04010400u);
        const kvc_h2 off = {(_Float16)-1152.f, (_Float16)-1152.f};
        mins = __builtin_bit_cast(uint32_t, __builtin_bit_cast(kvc_h2, biased) + off);                              // exact
        scales = raw.scw[s][0];
    } else {
        mins = kvc_half_pair((float)raw.min_int(s, 0, pmode), (float)raw.min_int(s, 1, pmode));                    // exact
        scales = raw.scale_bits(s, 0, pmode) | (raw.scale_bits(s, 1, pmode) << 16);
    }
}

// Which of the wave's operand-table slots serve a tile.  A V tile needs the tables of one head, or of two when its 64
// channels straddle a head boundary; consecutive tiles of a row share heads (head_dim 128: two tiles per head;
// head_dim 96: three tiles over two heads), and a head's tables -- the softmax of its 128 scores, the weights split into
// fp16 parts, the tokens' minima and scales -- are the same for every tile.  So a wave that works through a run of tiles
// keeps what it has built: KvcTableState says which head each slot holds, kvc_plan_tables which slot a tile's first head
// uses (the second head's is the other one) and which heads still have to be built.  Rounded mode only (the other
// arithmetic folds per-tile constants into its tables); K tiles change head, or block of channel parameters, every tile.
// (Plain integers picked with selects, no arrays: an array indexed by a run-time slot number would live in scratch memory.)
struct KvcTableState {
    int head0, head1;         // batch entry * kv_heads + head whose tables lie in slot 0 / 1, -1: none
    int row;                  // tile row they were built for
    int lo0, lo1;             // the slot's low-part columns hold something
    __device__ __forceinline__ int head(int slot) const { return slot ? head1 : head0; }
    __device__ __forceinline__ int lo(int slot) const { return slot ? lo1 : lo0; }
    __device__ __forceinline__ void set_head(int slot, int h)
    {
        head0 = slot ? head0 : h;
        head1 = slot ? h : head1;
    }
    __device__ __forceinline__ void set_lo(int slot, int v)
    {
        lo0 = slot ? lo0 : v;
        lo1 = slot ? v : lo1;
    }
};

struct KvcTablePlan {
    int slot0;                // table slot of the tile's first head
    int build;                // bit s set: head s of the tile (0: first, 1: second) has to be built
    int straddles;
};

template <int KIND, bool ROUNDED>
__device__ __forceinline__ KvcTablePlan kvc_plan_tables(const KvcFusedArgs &a, const KvcTilePos &p, KvcTableState &st)
{
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    KvcTablePlan pl;
    pl.slot0 = 0;
    pl.straddles = (SLOTS == 2 && p.d0 + KVC_WAVE > a.head_dim) ? 1 : 0;
    pl.build = pl.straddles ? 3 : 1;
    if constexpr (KIND != 0 && ROUNDED) {
        const bool same_row = st.row == p.row;
        const int hA = p.b * a.kv_heads + p.h;
        if constexpr (SLOTS == 1) {
            if (same_row && st.head0 == hA) pl.build = 0;
            st.head0 = hA;
        } else {
            int b2, h2;
            kvc_second_head(a, p, b2, h2);
            const int hB = pl.straddles ? b2 * a.kv_heads + h2 : -2;
            const bool in0 = same_row && st.head0 == hA, in1 = same_row && st.head1 == hA;
            const bool buildA = !in0 && !in1;
            // a head that has to be built leaves the second head's tables where they are
            const int sA = in0 ? 0 : in1 ? 1 : (same_row && st.head0 == hB) ? 1 : 0;
            const int sB = 1 - sA;
            const bool buildB = pl.straddles && !(same_row && st.head(sB) == hB);
            pl.slot0 = sA;
            pl.build = (buildA ? 1 : 0) | (buildB ? 2 : 0);
            if (!same_row) st.head0 = st.head1 = -1;
            st.set_head(sA, hA);
            if (pl.straddles) st.set_head(sB, hB);
        }
        st.row = p.row;
    }
    return pl;
}

// Build those operand tables of a fetched tile that the plan asks for; returns per query head the constant term
// sum_i min_i weight_i of this lane's head (zero in rounded mode) and the power of two the weights were divided by to
// stay inside fp16; sel_out: 1 for a lane whose channel lies past the tile's head boundary.
template <int REP, int KIND, bool ROUNDED>
__device__ __forceinline__ void kvc_mfma_stage_ops(const KvcFusedArgs &a, const KvcTilePos &pos, const KvcTablePlan &pl, int lane,
                                                   const KvcRaw<REP, KvcGeom<KIND>::SLOTS, KvcGeom<KIND>::XW> &raw,
                                                   uint32_t *btab, uint32_t *mstab, float (&bias)[REP], float &unscale,
                                                   int &sel_out, KvcTableState &st)
{
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    constexpr int NM = kvc_mfma_sets(REP);
    using T = KvcMfmaTables<REP>;
    const int D = a.head_dim;
    const int row = pos.row;
    float bias_s[SLOTS][REP];
    float v[SLOTS][REP][2];
    const bool live = KIND != 0 || 2 * lane < D;
    const int pmode0 = kvc_pair_mode<KIND>(a);
    // (the second head's parameters are always held as one word of scales and one of minima: copies of the first
    // head's where they are per token, fetched late and packed by the kernel otherwise)
    auto pmode_of = [&](int s) { return s == 0 ? pmode0 : (int)KVC_PAIR_ADJACENT; };
    int sel = 0;
    if (SLOTS == 2) sel = (pos.d0 + lane) >= D;                               // 1 past a head boundary
    sel_out = sel;
    auto slot_of = [&](int s) { return s == 0 ? pl.slot0 : 1 - pl.slot0; };   // table slot of the tile's head s
    // Rounded mode without the softmax: the weights are the caller's fp16 values (q, or p).  Unless one of them is
    // subnormal they are their own high parts and the low parts are zero: the words go to the table as they were
    // loaded, and the low columns stay (or are made) zero.
    if constexpr (ROUNDED && !KvcGeom<KIND>::SOFTMAX) {
        bool subnormal = false;
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            if (!((pl.build >> s) & 1)) continue;
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const kvc_h2 w = __builtin_bit_cast(kvc_h2, raw.x[s][r][0]);
                subnormal = subnormal | __builtin_amdgcn_classh(w.x, 0x90) | __builtin_amdgcn_classh(w.y, 0x90);
            }
        }
        if (!__any(live && subnormal)) {
            const int g = lane >> 1, odd = lane & 1;
#pragma unroll
            for (int s = 0; s < SLOTS; s++) {
                if (!((pl.build >> s) & 1)) continue;
                const int ts = slot_of(s);
                if (live) {
                    uint32_t *bg = btab + ts * T::BTAB_SLOT_WORDS + g * (NM * 8) + odd;
                    if (st.lo(ts)) {                           // low parts an earlier tile of this wave left there
#pragma unroll
                        for (int r = 0; r < REP; r++) bg[(((2 * r + 1) >> 2) * 4 + ((2 * r + 1) & 3)) * 2] = 0u;
                    }
#pragma unroll
                    for (int r = 0; r < REP; r++) bg[(((2 * r) >> 2) * 4 + ((2 * r) & 3)) * 2] = raw.x[s][r][0];
                    uint32_t *mg = mstab + ts * T::MSTAB_SLOT_WORDS + g * 4 + odd;
                    kvc_mfma_min_scale_words(raw, s, pmode_of(s), mg[0], mg[2]);
                }
                st.set_lo(ts, 0);
            }
            unscale = 1.f;
#pragma unroll
            for (int r = 0; r < REP; r++) bias[r] = 0.f;
            return;
        }
    }
    float vmax = 0.f;
#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
#pragma unroll
        for (int r = 0; r < REP; r++) bias_s[s][r] = 0.f, v[s][r][0] = v[s][r][1] = 0.f;
        if (!((pl.build >> s) & 1)) continue;                  // no lane of this tile belongs to a second head, or the head's tables are there
        st.set_lo(slot_of(s), 1);
        int hb = pos.b, hh = pos.h;
        if (s == 1) kvc_second_head(a, pos, hb, hh);
#pragma unroll
        for (int r = 0; r < REP; r++) {
            float w0, w1;                                      // the two elements' weights: q, p, or exp(score - max)
            if (KvcGeom<KIND>::SOFTMAX) {
                const float s0 = __uint_as_float(raw.x[s][r][0]) * a.sm_scale;
                const float s1 = __uint_as_float(raw.x[s][r][KvcGeom<KIND>::XW - 1]) * a.sm_scale;
                const float m = kvc_wave_fmax_dpp(fmaxf(s0, s1));
                w0 = __expf(s0 - m);
                w1 = __expf(s1 - m);
                const float l = kvc_wave_sum_dpp(w0 + w1);
                if (lane == 0) {
                    float *ml = a.ml + (((int64_t)row * a.batch + hb) * a.q_heads + hh * REP + r) * 2;
                    ml[0] = m;     // tiles that share a head write the same pair
                    ml[1] = l;
                }
            } else {
                w0 = kvc_half_bits_to_float(raw.x[s][r][0] & 0xffffu);
                w1 = kvc_half_bits_to_float(raw.x[s][r][0] >> 16);
            }
            if (ROUNDED) {
                v[s][r][0] = w0;
                v[s][r][1] = w1;
            } else {
                const float sc0 = live ? kvc_half_bits_to_float(raw.scale_bits(s, 0, pmode_of(s))) : 0.f;
                const float sc1 = live ? kvc_half_bits_to_float(raw.scale_bits(s, 1, pmode_of(s))) : 0.f;
                v[s][r][0] = sc0 * w0;
                v[s][r][1] = sc1 * w1;
                bias_s[s][r] = (float)raw.min_int(s, 0, pmode_of(s)) * v[s][r][0] + (float)raw.min_int(s, 1, pmode_of(s)) * v[s][r][1];
                vmax = fmaxf(vmax, fmaxf(fabsf(v[s][r][0]), fabsf(v[s][r][1])));
            }
        }
        if (!ROUNDED) {
#pragma unroll
            for (int r = 0; r < REP; r++) bias_s[s][r] = kvc_wave_sum_dpp(bias_s[s][r]);
        }
    }
    // weights beyond fp16's range (never with sane scales): divide the tile's weights by a power of two
    float down = 1.f;
    unscale = 1.f;
    if (!ROUNDED && __any(!(vmax < 32768.f))) {
        const float m = kvc_wave_fmax_dpp(vmax);
        if (m < INFINITY) {                                    // otherwise the result is not finite either way
            int e;
            (void)frexpf(m, &e);                               // m < 2^e
            down = ldexpf(1.f, 14 - e);
            unscale = ldexpf(1.f, e - 14);
        }
    }
    const int g = lane >> 1, odd = lane & 1;
    if (live) {
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            if (!((pl.build >> s) & 1)) continue;
            const int ts = slot_of(s);
#pragma unroll
            for (int r = 0; r < REP; r++) {
                float h0, l0, h1, l1;
                kvc_split_weight(v[s][r][0] * down, h0, l0);
                kvc_split_weight(v[s][r][1] * down, h1, l1);
                const int c_hi = 2 * r, c_lo = 2 * r + 1;
                uint32_t *bg = btab + ts * T::BTAB_SLOT_WORDS + g * (NM * 8) + odd;
                bg[((c_hi >> 2) * 4 + (c_hi & 3)) * 2] = kvc_half_pair(h0, h1);
                bg[((c_lo >> 2) * 4 + (c_lo & 3)) * 2] = kvc_half_pair(l0, l1);
            }
            if (ROUNDED) {
                uint32_t *mg = mstab + ts * T::MSTAB_SLOT_WORDS + g * 4 + odd;
                kvc_mfma_min_scale_words(raw, s, pmode_of(s), mg[0], mg[2]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < REP; r++) bias[r] = (SLOTS == 2 && sel) ? bias_s[SLOTS - 1][r] : bias_s[0][r];
}

// -- decode loops -------------------------------------------------------------------------------------
// 2 G symbols per refill of 64 stream bits (G from each half window; 2 G a multiple of four), n a multiple of 2 G.
// bptr: LDS byte address of this lane's column in the operand table of the group the loop starts with;
// msptr: of that group's minima and scales (rounded mode).  Both advance with the groups consumed.
// HALF: two-byte table entries {symbol as fp16 | code length in the bits that symbols below 64 leave clear}: a table of
// 64 entries then fills 32 words, one per LDS bank, and two lanes that read different entries of one bank read the same
// word, which the LDS serves in one cycle (with four-byte entries a 64-entry table has two words per bank and 42 % of
// its LDS cycles are bank conflicts).  Costs an instruction per two symbols (join and mask instead of a byte permute);
// the lengths of a half window (at most 4 x 7 bits) are summed in five bits, above which symbol bits pile up.
template <int G, bool SKEW, int NM, bool ROUNDED, bool BCAST, bool HALF = false>
__device__ __forceinline__ void kvc_mfma_dot(uint32_t sbase, uint32_t &u, uint32_t fe, uint32_t mask4, int n,
                                             uint32_t &bptr, uint32_t &msptr, kvc_f4 (&acc)[NM], bool holder)
{
    static_assert((2 * G) % 4 == 0, "whole groups of four per refill");
    static_assert(!HALF || G <= 4, "the lengths of a half window must fit five bits");
    asm volatile("" : "+v"(msptr));      // kept in a vector register: one add per round instead of a move per read
    for (int i = 0; i < n; i += 2 * G) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0, used1 = 0;
        uint32_t e[2 * G];
        kvc_static_for<2 * G>([&](auto g_) {
            constexpr int g = decltype(g_)::value;
            if (g == G) {
                R = __builtin_amdgcn_alignbit(hi, lo, es);       // (shifts by the low five bits of es)
                if (HALF) used1 = es & 31u, es = 0;
            }
            if constexpr (HALF) e[g] = *(const kvc_lds_u16 *)(uintptr_t)((R & mask4) | fe);
            else e[g] = *(const kvc_lds_u32 *)(uintptr_t)((R & mask4) | fe);
            if (g != G - 1 && g != 2 * G - 1) R = __builtin_amdgcn_alignbit(R, R, e[g]);
            es += e[g];
            if constexpr (g % 4 == 3) {
                constexpr int q = g / 4;
                uint32_t a01, a23;
                if constexpr (HALF) {
                    a01 = ((e[g - 2] << 16) | e[g - 3]) & 0xffe0ffe0u;
                    a23 = ((e[g] << 16) | e[g - 1]) & 0xffe0ffe0u;
                } else {
                    a01 = kvc_pack_hi16(e[g - 3], e[g - 2]);
                    a23 = kvc_pack_hi16(e[g - 1], e[g]);
                }
                if (ROUNDED) {
                    const kvc_w4 ms = *(const kvc_lds_w4 *)(uintptr_t)(msptr + q * 16);
                    a01 = kvc_dequant_pair(a01, ms.x, ms.z);
                    a23 = kvc_dequant_pair(a23, ms.y, ms.w);
                }
#pragma unroll
                for (int s = 0; s < NM; s++)
                    acc[s] = kvc_mfma4<BCAST>(a01, a23, kvc_read_columns<BCAST>(bptr + (q * NM + s) * 32, holder), acc[s]);
            }
        });
        u += HALF ? used1 + (es & 31u) : es & 0xffu;
        bptr += (2 * G / 4) * NM * 32;
        msptr += (2 * G / 4) * 16;
    }
}

// Two symbols per look-up: PG pairs from each half window, 4 PG symbols per refill; n a multiple of 4 PG.
template <int PG, bool SKEW, int NM, bool ROUNDED, bool BCAST>
__device__ __forceinline__ void kvc_mfma_pair_dot(uint32_t sbase, uint32_t &u, uint32_t fe, uint32_t maskp, int n,
                                                  uint32_t &bptr, uint32_t &msptr, kvc_f4 (&acc)[NM], bool holder)
{
    asm volatile("" : "+v"(msptr));      // kept in a vector register: one add per round instead of a move per read
    for (int i = 0; i < n; i += 4 * PG) {
        const kvc_lds_word *wp = (const kvc_lds_word *)(uintptr_t)kvc_refill_address<SKEW>(sbase, u);
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2];
        const uint32_t lo = __builtin_amdgcn_alignbit(w1, w0, u), hi = __builtin_amdgcn_alignbit(w2, w1, u);
        uint32_t R = lo, es = 0, used1 = 0;
        uint32_t e[2 * PG];
        kvc_static_for<2 * PG>([&](auto p_) {
            constexpr int p = decltype(p_)::value;
            if (p == PG) {
                used1 = es & KVC_PAIR_LEN_MASK;                 // at most 30: the sum of a half window fits the field
                R = __builtin_amdgcn_alignbit(hi, lo, used1);
                es = 0;
            }
            e[p] = *(const kvc_lds_u32 *)(uintptr_t)((R & maskp) | fe);
            if (p != PG - 1 && p != 2 * PG - 1) R = __builtin_amdgcn_alignbit(R, R, e[p]);
            es += e[p];
            if constexpr (p % 2 == 1) {
                constexpr int q = p / 2;
                uint32_t a01 = e[p - 1] & ~KVC_PAIR_LEN_MASK, a23 = e[p] & ~KVC_PAIR_LEN_MASK;
                if (ROUNDED) {
                    const kvc_w4 ms = *(const kvc_lds_w4 *)(uintptr_t)(msptr + q * 16);
                    a01 = kvc_dequant_pair(a01, ms.x, ms.z);
                    a23 = kvc_dequant_pair(a23, ms.y, ms.w);
                }
#pragma unroll
                for (int s = 0; s < NM; s++)
                    acc[s] = kvc_mfma4<BCAST>(a01, a23, kvc_read_columns<BCAST>(bptr + (q * NM + s) * 32, holder), acc[s]);
            }
        });
        u += used1 + (es & KVC_PAIR_LEN_MASK);
        bptr += PG * NM * 32;
        msptr += PG * 16;
    }
}

// One symbol per refill, generic table and long-code list in global memory; words from LDS (staged, bit-reversed)
// or from global memory (raw, bounds-checked word by word).  Returns this lane's sums, one per query head.
template <int REP, bool GSRC, bool ROUNDED>
__device__ __noinline__ KvcVec<REP> kvc_mfma_slow_tile(const uint32_t *words, uint32_t nwords, uint32_t pos,
                                                       const uint32_t *__restrict__ lut_g, int n, const uint32_t *btab,
                                                       const uint32_t *mstab, uint32_t skew)
{
    constexpr int NM = kvc_mfma_sets(REP);
    const uint32_t lshift = 32u - lut_g[0], nlong = lut_g[2];
    const uint32_t *longs = lut_g + KVC_LUT_HEADER_WORDS;
    const uint32_t *entries = lut_g + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    const uint16_t *bh = reinterpret_cast<const uint16_t *>(btab), *mh = reinterpret_cast<const uint16_t *>(mstab);
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
        const int g = i >> 2, k = i & 3;
        float x = (float)sym;
        if (ROUNDED) {
            const uint32_t ms = (uint32_t)mh[g * 8 + k] | ((uint32_t)mh[g * 8 + 4 + k] << 16);
            x = kvc_rounded_value(__float2half_rn(x), ms);
        }
#pragma unroll
        for (int r = 0; r < REP; r++) {
            const int c_hi = 2 * r, c_lo = 2 * r + 1;
            const float whi = kvc_half_bits_to_float(bh[((g * NM + (c_hi >> 2)) * 4 + (c_hi & 3)) * 4 + k]);
            const float wlo = kvc_half_bits_to_float(bh[((g * NM + (c_lo >> 2)) * 4 + (c_lo & 3)) * 4 + k]);
            acc.v[r] = fmaf(x, whi + wlo * (1.f / KVC_LO_SCALE), acc.v[r]);
        }
        pos += len;
    }
    return acc;
}

// value of `v` in the next lane of the quad (lanes 1 and 3 read themselves)
__device__ __forceinline__ float kvc_quad_next(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xF5 /* quad_perm:[1,1,3,3] */, 0xf, 0xf, false));
}

template <int REP, int KIND, bool ROUNDED>
__global__ void __launch_bounds__(KVC_WG, kvc_fused_mfma_occupancy(REP, KIND)) kvc_fused_mfma_kernel(KvcFusedArgs a_in)
{
    const KvcFusedArgs &a = a_in;
    constexpr bool IS_K = KIND == 0;
    constexpr int SLOTS = KvcGeom<KIND>::SLOTS;
    constexpr int NM = kvc_mfma_sets(REP);
    using T = KvcMfmaTables<REP>;
    // dynamic LDS: the decode table (at offset 0, so that its address folds into the look-ups), then per wave:
    // operand tables, packed payload
    extern __shared__ __align__(16) uint32_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int D = a.head_dim;
    constexpr int OPS_WORDS = kvc_mfma_ops_words(SLOTS, REP, ROUNDED);
    const int per_wave = OPS_WORDS + a.pack_words;
    uint32_t *btab = smem + a.table_words + wave * per_wave;
    uint32_t *mstab = btab + SLOTS * T::BTAB_SLOT_WORDS;
    uint32_t *pack = btab + OPS_WORDS;
    // Which tiles this wave takes.  Plain launch: grid (column groups, tile rows), every wave `tiles_per_wave`
    // consecutive columns of its row.  Scheduled launch (sched_nseg > 0; one codebook for the whole stream): a 1-D grid
    // over the row-major tile sequence in a few segments, the waves of segment k taking sched_run[k] consecutive tiles
    // each; runs shorten towards the end of the launch, so that most tiles share a wave's set-up with several others
    // while the last workgroups to start are short and the chip drains quickly.
    int t_first, ntiles;
    const int cols = a.s.cols;
    if (a.sched_nseg) {
        const int wg = blockIdx.x;
        int k = 0;
#pragma unroll
        for (int i = 1; i < KVC_SCHED_SEGMENTS; i++)
            if (i < a.sched_nseg && wg >= a.sched_wg[i]) k = i;
        const int run = a.sched_run[k];
        t_first = a.sched_tile[k] + ((wg - a.sched_wg[k]) * KVC_WAVES_PER_WG + wave) * run;
        ntiles = a.sched_tile[k + 1] - t_first;
        ntiles = ntiles < run ? ntiles : run;
    } else {
        const int TPW = a.s.tiles_per_wave;
        const int c0 = (blockIdx.x * KVC_WAVES_PER_WG + wave) * TPW;
        t_first = blockIdx.y * cols + c0;
        ntiles = cols - c0;
        ntiles = ntiles < TPW ? ntiles : TPW;
    }
    int row = t_first / cols, col = t_first - row * cols;
    // block_info of the wave's j-th tile in lane j (asked for before the table is set up: the two waits overlap)
    uint32_t bi_off = 0, bi_bn = 0;
    if (lane < ntiles) {
        const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.s.block_infos + 8 * ((int64_t)t_first + lane));
        bi_off = bi[0];
        bi_bn = bi[1];
    }
    const int64_t cb = a.s.rows_per_codebook ? (a.sched_nseg ? 0 : (int)blockIdx.y) / a.s.rows_per_codebook : 0;
    const uint32_t *__restrict__ lut_g = a.s.luts + cb * KVC_LUT_WORDS;
    const uint32_t lbits = lut_g[0], lmax = lut_g[1], nlong = lut_g[2];
    const bool fast_book = nlong == 0 && lmax >= 1u && lmax <= 7u && (1u << lbits) <= (uint32_t)a.table_words;
    // one-symbol entries: the symbol as fp16 in the upper half, the code length (never beyond the index width, which
    // bounds how far a corrupt stream can run) in the lowest byte
    auto fentry = [&](uint32_t i) {
        const uint32_t e = lut_g[KVC_LUT_FENTRY_OFFSET + i];
        const uint32_t len = (e & 0xffu) > lbits ? lbits : (e & 0xffu);
        return ((uint32_t)__half_as_ushort(__float2half_rn(__uint_as_float(e & 0xffffff00u))) << 16) | len;
    };
    const uint32_t pbits = 2u * lmax;
    // two symbols per look-up: twice the longest code fits the index, and no symbol's fp16 pattern needs the five
    // bits the lengths of a two-symbol entry go to (header word 6: OR of all the patterns)
    const bool pairs = fast_book && a.pair_bits != 0 && pbits <= (uint32_t)a.pair_bits && pbits <= 10u &&
                       (1u << pbits) <= (uint32_t)a.table_words && (lut_g[6] & KVC_PAIR_LEN_MASK) == 0u;
    // codes of 6 or 7 bits: two-byte entries (see kvc_mfma_dot), where no symbol's fp16 pattern needs its five lowest bits.
    // Not for V tiles that may straddle two heads: with that loop beside the others the kernel needs one register more
    // than six waves per SIMD leave it, and the compiler then spills in the per-tile path of every variant.
    constexpr bool HALF_OK = SLOTS == 1;
    const bool half_table = HALF_OK && fast_book && !pairs && lbits >= 6u && a.half_table != 0 && (lut_g[6] & KVC_PAIR_LEN_MASK) == 0u;
    const uint32_t lead_bits = half_table ? 1u : 2u;                   // bits of the window below the table index
    if (pairs) {
        // the one-symbol table goes to the (not yet used) per-wave areas; the two-symbol table is derived from it
        uint32_t *tmp = smem + a.table_words;
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) tmp[i] = fentry(i);
        __syncthreads();
        const uint32_t m1 = (1u << lbits) - 1u;
        for (uint32_t idx = tid; idx < (1u << pbits); idx += KVC_WG) {
            const uint32_t e0 = tmp[idx & m1];
            const uint32_t e1 = tmp[(idx >> (e0 & 0xffu)) & m1];
            smem[idx] = (e1 & 0xffff0000u) | (e0 >> 16) | ((e0 & 0xffu) + (e1 & 0xffu));
        }
        __syncthreads();
    } else if (half_table) {
        uint16_t *t16 = reinterpret_cast<uint16_t *>(smem);
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) {
            const uint32_t e = fentry(i);
            t16[i] = (uint16_t)((e >> 16) | (e & 0xffu));
        }
    } else if (fast_book) {
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) smem[i] = fentry(i);
    }
    // columns that no query head owns (REP 1: columns 2 and 3) are multiplied too: give them zeros once
    for (int i = lane; i < SLOTS * T::BTAB_SLOT_WORDS; i += KVC_WAVE) btab[i] = 0;
    if (lane < KVC_PACK_LEAD) pack[lane] = 0;
    __syncthreads();
    const uint32_t mask4 = ((1u << lbits) - 1u) << lead_bits, maskp = ((1u << pbits) - 1u) << 2;
    const int n = IS_K ? D : KVC_V_TOKENS;                             // symbols per lane stream
    // symbols per refill in the main part (a multiple of four); what is left goes eight per refill
    const int per = pairs ? (pbits <= 7u ? 16 : 12) : (lmax <= 3u ? 16 : lmax <= 5u ? 12 : 8);
    int n_main = (n / per) * per;
    while ((n - n_main) % 8 != 0) n_main -= per;
    const uint32_t fe = kvc_lds_addr(smem);                            // 0: the table opens the workgroup's LDS

    if (ntiles <= 0) return;
    KvcRaw<REP, SLOTS, KvcGeom<KIND>::XW> raw;
    // (the one place where the tile's batch entry, head and channel offset are worked out by division)
    KvcTilePos pos = kvc_tile_pos<IS_K>(a, row, col);
    KvcTableState tabs;
    tabs.head0 = tabs.head1 = tabs.row = -1;
    tabs.lo0 = tabs.lo1 = 0;                                             // (the low-part columns start as zeros)
    KvcTablePlan plan = kvc_plan_tables<KIND, ROUNDED>(a, pos, tabs);
    kvc_fetch_tile<REP, KIND, 0, SLOTS == 2>(a, pos, __builtin_amdgcn_readlane(bi_off, 0), __builtin_amdgcn_readlane(bi_bn, 0), lane, raw);
    // the second head's parameters where every token has groups of its own per batch entry or head: fetched only now
    auto late_params = [&](const KvcFusedArgs &a, const KvcTilePos &p, const KvcTablePlan &pl, int lane) {
        if constexpr (SLOTS == 2) {
            if ((pl.build & 2) && kvc_pair_mode<KIND>(a) != KVC_PAIR_ADJACENT) {
                int b2, h2;
                kvc_second_head(a, p, b2, h2);
                kvc_fetch_separate_params(a, p.row, b2, h2, lane, 1, raw);
                // ... and kept in the form of parameters that lie next to each other: two registers instead of four
                raw.scw[1][0] = (raw.scw[1][0] & 0xffffu) | (raw.scw[1][1] << 16);
                raw.mnw[1][0] = (raw.mnw[1][0] & 0xffu) | ((raw.mnw[1][1] & 0xffu) << 8);
            }
        }
    };
    late_params(a, pos, plan, lane);
    float bias[REP], unscale;
    int sel = 0;
    uint32_t first, longest;
    KvcStaged st = kvc_stage_payload(a, lane, raw, pack, first, longest);
    if (st.fits) st.u0 = 32u * KVC_PACK_LEAD + first * 8u - lead_bits;       // one or two bits before the lane's first code
    kvc_mfma_stage_ops<REP, KIND, ROUNDED>(a, pos, plan, lane, raw, btab, mstab, bias, unscale, sel, tabs);
    kvc_wave_sync();
    for (int it = 0; it < ntiles; it++) {
        // the arguments are read again per tile rather than kept in scalar registers through the decode loops (the
        // kernel needs more scalars than there are registers, and every spilled one costs a vector instruction)
        const KvcFusedArgs &a = kvc_kernarg_again<KvcFusedArgs>();
        const bool more = it + 1 < ntiles;
        const KvcTilePos pos_next = kvc_tile_after<IS_K>(a, pos);          // row-major successor
        // which of the wave's operand tables the next tile can use as they are: it then needs no weights
        KvcTablePlan plan_next = plan;
        if (more) plan_next = kvc_plan_tables<KIND, ROUNDED>(a, pos_next, tabs);
        // the lane number is made opaque per tile, so that the addresses the fetch and the staging derive from it
        // are not kept in registers through the decode loops
        int lane_f = lane;
        asm volatile("" : "+v"(lane_f));
        if (more)   // loads for the next tile fly while this one is decoded
            kvc_fetch_tile<REP, KIND, 0, SLOTS == 2>(a, pos_next, __builtin_amdgcn_readlane(bi_off, it + 1),
                                                     __builtin_amdgcn_readlane(bi_bn, it + 1), lane_f, raw, ~plan_next.build);
        const int my_slot = sel ? 1 - plan.slot0 : plan.slot0;
        const uint32_t *my_btab = btab + my_slot * T::BTAB_SLOT_WORDS, *my_mstab = mstab + my_slot * T::MSTAB_SLOT_WORDS;
        // (wave-uniform: some low-part column of the tables this tile reads holds something)
        bool lo_used = tabs.lo(plan.slot0) != 0;
        if constexpr (SLOTS == 2) lo_used = lo_used || (plan.straddles && tabs.lo(1 - plan.slot0) != 0);
        // geometry of the results
        int64_t out_base, out_step;
        if (IS_K) {
            out_base = ((int64_t)pos.b * a.q_heads + pos.h * REP) * a.out_stride + (int64_t)pos.row * KVC_WAVE;
            out_step = a.out_stride;
        } else {
            int b = pos.b, h = pos.h;
            if (sel) kvc_second_head(a, pos, b, h);                     // the next head may open the next batch entry
            out_base = (((int64_t)pos.row * a.batch + b) * a.q_heads + h * REP) * D + (pos.d0 - sel * D);
            out_step = D;
        }
        if (fast_book && st.fits) {
            kvc_f4 acc[NM];
#pragma unroll
            for (int s = 0; s < NM; s++) acc[s] = kvc_f4{0.f, 0.f, 0.f, 0.f};
            uint32_t u = st.u0;
            uint32_t bptr = kvc_lds_addr(my_btab) + (lane & 3) * 8, msptr = kvc_lds_addr(my_mstab);
            const uint32_t sbase = kvc_lds_addr(pack);
            // one head per tile: all sixteen blocks share their operand columns, which lanes 0 - 15 then hold for all
            constexpr bool BCAST = SLOTS == 1;
            const bool holder = lane < 16;
            auto run = [&](auto skew_) {
                constexpr bool SK = decltype(skew_)::value;
                if (pairs) {
                    if (per == 16) kvc_mfma_pair_dot<4, SK, NM, ROUNDED, BCAST>(sbase, u, fe, maskp, n_main, bptr, msptr, acc, holder);
                    else kvc_mfma_pair_dot<3, SK, NM, ROUNDED, BCAST>(sbase, u, fe, maskp, n_main, bptr, msptr, acc, holder);
                    if (n - n_main) kvc_mfma_pair_dot<2, SK, NM, ROUNDED, BCAST>(sbase, u, fe, maskp, n - n_main, bptr, msptr, acc, holder);
                } else {
                    if (per == 16) kvc_mfma_dot<8, SK, NM, ROUNDED, BCAST>(sbase, u, fe, mask4, n_main, bptr, msptr, acc, holder);
                    else if (per == 12) kvc_mfma_dot<6, SK, NM, ROUNDED, BCAST>(sbase, u, fe, mask4, n_main, bptr, msptr, acc, holder);
                    const int rest = per == 8 ? n : n - n_main;
                    if (HALF_OK && rest && half_table) kvc_mfma_dot<4, SK, NM, ROUNDED, BCAST, HALF_OK>(sbase, u, fe, mask4, rest, bptr, msptr, acc, holder);
                    else if (rest) kvc_mfma_dot<4, SK, NM, ROUNDED, BCAST>(sbase, u, fe, mask4, rest, bptr, msptr, acc, holder);
                }
            };
            if (a.skew) run(std::true_type{});
            else run(std::false_type{});
            // register i of lane 4 b + j: row 4 b + i, column 4 set + j; the even columns take their low parts from
            // the lane to their right and carry the results of query head 2 set + j / 2
            int lane_e = lane;
            // (one query head: nothing derived from the lane number is kept across the decode loops, which lets the
            // single-head V kernel fit the registers of seven waves; with more heads the kernels measured no better for it)
            if constexpr (REP == 1) asm volatile("" : "+v"(lane_e));
            const int j = lane_e & 3, rows4 = (lane_e >> 2) * 4;
#pragma unroll
            for (int s = 0; s < NM; s++) {
                float res[4];
                const int r = 2 * s + (j >> 1);
                float bs = 0.f;
#pragma unroll
                for (int rr = 0; rr < REP; rr++)
                    if (rr == r) bs = bias[rr];
#pragma unroll
                for (int i = 0; i < 4; i++) res[i] = acc[s][i];
                if (lo_used) {
#pragma unroll
                    for (int i = 0; i < 4; i++) res[i] = fmaf(kvc_quad_next(acc[s][i]), 1.f / KVC_LO_SCALE, acc[s][i]);
                }
                if (!ROUNDED) {                        // rounded mode folds nothing into a constant and never rescales
#pragma unroll
                    for (int i = 0; i < 4; i++) res[i] = res[i] * unscale + bs;
                }
                if ((j & 1) == 0 && r < REP) {
                    const int64_t o = out_base + r * out_step + rows4;
                    if (a.out_f32) {
                        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.out) + o) = make_float4(res[0], res[1], res[2], res[3]);
                    } else {
                        const uint32_t h01 = kvc_half_pair(res[0], res[1]), h23 = kvc_half_pair(res[2], res[3]);
                        *reinterpret_cast<uint2 *>(reinterpret_cast<__half *>(a.out) + o) = make_uint2(h01, h23);
                    }
                }
            }
        } else {
            KvcVec<REP> res;
            if (st.fits)
                res = kvc_mfma_slow_tile<REP, false, ROUNDED>(pack, (uint32_t)a.pack_logical, st.u0 + lead_bits, lut_g, n, my_btab,
                                                              my_mstab, (uint32_t)a.skew);
            else
                res = kvc_mfma_slow_tile<REP, true, ROUNDED>(st.gwords, st.gnwords, st.gpos, lut_g, n, my_btab, my_mstab, 0u);
            // here a lane holds the results of its own row; in a V tile every lane's head slot is its block's
            int lane_o = lane;
            if constexpr (REP == 1) asm volatile("" : "+v"(lane_o));
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const int64_t o = out_base + r * out_step + lane_o;
                const float v = res.v[r] * unscale + bias[r];
                if (a.out_f32) reinterpret_cast<float *>(a.out)[o] = v;
                else reinterpret_cast<__half *>(a.out)[o] = __float2half(v);
            }
        }
        if (more) {
            kvc_wave_sync();     // every lane is done reading this tile's LDS data
            int lane_s = lane;
            asm volatile("" : "+v"(lane_s));
            st = kvc_stage_payload(a, lane_s, raw, pack, first, longest);
            if (st.fits) st.u0 = 32u * KVC_PACK_LEAD + first * 8u - lead_bits;
            late_params(a, pos_next, plan_next, lane_s);
            kvc_mfma_stage_ops<REP, KIND, ROUNDED>(a, pos_next, plan_next, lane_s, raw, btab, mstab, bias, unscale, sel, tabs);
            kvc_wave_sync();
        }
        pos = pos_next;
        plan = plan_next;
    }
}

