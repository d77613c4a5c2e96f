/*
 * kvc_oracle.c -- CPU restatement of the KVComp codec path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it.  The shipped library (kvcomp_amd/lib/libkvcomp_hip.so)
 * never links, calls or falls back to anything in this directory.
 *
 * Every function restates, in plain scalar C, the algorithm of the reference file:line it cites
 * (paths relative to the reference checkout).  Nothing here is copied from the reference; the
 * control flow is deliberately the simplest one that yields the same bytes.
 *
 * Pinning status of each function (what independent evidence fixes its output):
 *   kvo_h2f / kvo_f2h        exhaustive / randomized comparison with numpy float16 conversion.
 *   kvo_quant / kvo_dequant  bit-for-bit against stock PyTorch CPU fp16 ops (min/max/sub/mul/div/round),
 *                            invariants (min symbol 0, 0.53*scale error bound), hand-worked cases.
 *   kvo_huffman_build        Python stdlib heapq driven by a frequency-only comparison (same pop order),
 *                            Kraft equality, optimal cost vs. an independent O(n^2) Huffman, closed
 *                            forms (2 symbols, equal counts over 2^k symbols), and -- where it builds --
 *                            the reference's own huffman.cpp compiled into oracle/_ref.
 *   kvo_encode_table / kvo_decode_tree
 *                            hand-worked byte vectors, tree-walk-reaches-leaf property, oracle/_ref.
 *   kvo_encode_tiles / kvo_decode_tiles
 *                            hand-worked one-tile example (2- and 3-symbol codebooks), independent
 *                            bit-string model in Python, exact round trip.  The reference's CUDA kernels
 *                            cannot run in this environment, so the tile wire format rests on these.
 *   kvo_huffman_bits         independent Python bit-string model (str.join of code strings).
 *   kvo_fused_k / kvo_fused_v  double-precision sums of the dequantized fp16 cache; compared with fp32
 *                            PyTorch matmul in the tests.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define KVO_VEC_PER_TILE 64   /* include/kernels.h:13,18  K_VEC_PER_BLK = V_VEC_PER_BLK = 64 */

/* ------------------------------------------------------------------------------------------ */
/* IEEE binary16 <-> binary32, round-to-nearest-even (what every fp16 PyTorch CPU op does      */
/* around its fp32 "opmath").                                                                  */
/* ------------------------------------------------------------------------------------------ */
float kvo_h2f(uint16_t h)
{
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, u;
    if (e == 0) {
        if (m == 0) {
            u = s;
        } else {                       /* subnormal half = m * 2^-24: normalise */
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            u = s | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13);
        }
    } else if (e == 31) {
        u = s | 0x7f800000u | (m << 13);
    } else {
        u = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t kvo_f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) {            /* inf / nan */
        if (x == 0x7f800000u) return sign | 0x7c00u;
        return sign | 0x7c00u | 0x200u | (uint16_t)((x >> 13) & 0x3ffu);
    }
    if (x >= 0x477ff000u) return sign | 0x7c00u;      /* >= 65520 rounds to inf */
    if (x <= 0x33000000u) return sign;                 /* <= 2^-25 rounds to (signed) zero */
    if (x < 0x38800000u) {             /* result is a subnormal half */
        int e = (int)(x >> 23);
        uint32_t m = (x & 0x7fffffu) | 0x800000u;
        int sh = 126 - e;              /* 14..24 */
        uint32_t r = m >> sh, rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return sign | (uint16_t)r;
    }
    uint32_t r = x + 0xfffu + ((x >> 13) & 1u);
    return sign | (uint16_t)((r - 0x38000000u) >> 13);
}

/* ------------------------------------------------------------------------------------------ */
/* Q1  error-bounded block quantizer.                                                          */
/*     utils/compute.py:93-106 (quant), :74-91 (quant_ints); src/compute.cpp:40-58.            */
/*                                                                                             */
/* Tensor is fp16 [NB, BS, B, H, D] contiguous (models/cache/kvcomp_encode.py:83).  A group    */
/* is the set of elements that share (min, scale); reduce_mask bit k set means dimension k of  */
/* (BS=bit0, B=bit1, H=bit2, D=bit3) is reduced over.  The reference's modes are:              */
/*   kernel path K BlockQuant  dims [1,2,3,4] -> mask 0xF   (kvcomp_encode.py:10-13)           */
/*   kernel path V TokenQuant  dims [2,3,4]   -> mask 0xE                                      */
/*   ChannelQuant (utils/compute.py:140, per (b,h,block,channel)) -> mask 0x1                  */
/*   sim TokenQuant (utils/compute.py:141, per (b,block,token))   -> mask 0xC                  */
/*   VectorQuant (utils/compute.py:142)                            -> mask 0x8                  */
/*   sim BlockQuant (utils/compute.py:139, per (b,block))          -> mask 0xD                  */
/*                                                                                             */
/* Arithmetic, one fp16 PyTorch op per line (each = fp32 op then RN16):                        */
/*   range = RN16(max - min); scale = RN16(f32(range) * f32(eb))                               */
/*   min_i = rint(RN16(f32(min) / f32(scale)))                                                 */
/*   q     = rint(RN16(f32(x)   / f32(scale)));  sym = RN16(q - min_i)                         */
/* Outputs are the fp16 tensors the reference returns plus the .to(uint8)/.to(int8) casts of   */
/* kvcomp_encode.py:97-98 (defined here only for values already in range).                     */
/* ------------------------------------------------------------------------------------------ */
static inline int64_t kvo_group_index(int64_t nb, int64_t bs, int64_t b, int64_t h, int64_t d,
                                      int64_t BS, int64_t B, int64_t H, int64_t D, int mask)
{
    int64_t gBS = (mask & 1) ? 1 : BS, gB = (mask & 2) ? 1 : B, gH = (mask & 4) ? 1 : H, gD = (mask & 8) ? 1 : D;
    int64_t bs_ = (mask & 1) ? 0 : bs, b_ = (mask & 2) ? 0 : b, h_ = (mask & 4) ? 0 : h, d_ = (mask & 8) ? 0 : d;
    return (((nb * gBS + bs_) * gB + b_) * gH + h_) * gD + d_;
}

int64_t kvo_quant_groups(int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int mask)
{
    return NB * ((mask & 1) ? 1 : BS) * ((mask & 2) ? 1 : B) * ((mask & 4) ? 1 : H) * ((mask & 8) ? 1 : D);
}

/* less-than / greater-than on halves through their exact float values */
int kvo_quant(const uint16_t *x, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int mask, float eb,
              uint16_t *sym_f16, uint16_t *min_f16, uint16_t *scale_f16, uint8_t *sym_u8, int8_t *min_i8)
{
    int64_t G = kvo_quant_groups(NB, BS, B, H, D, mask);
    float *gmin = (float *)malloc(sizeof(float) * (size_t)G);
    float *gmax = (float *)malloc(sizeof(float) * (size_t)G);
    if (!gmin || !gmax) { free(gmin); free(gmax); return -1; }
    for (int64_t g = 0; g < G; g++) { gmin[g] = INFINITY; gmax[g] = -INFINITY; }
    int64_t idx = 0;
    for (int64_t nb = 0; nb < NB; nb++)
      for (int64_t bs = 0; bs < BS; bs++)
        for (int64_t b = 0; b < B; b++)
          for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++, idx++) {
                float v = kvo_h2f(x[idx]);
                int64_t g = kvo_group_index(nb, bs, b, h, d, BS, B, H, D, mask);
                if (v < gmin[g]) gmin[g] = v;
                if (v > gmax[g]) gmax[g] = v;
            }
    for (int64_t g = 0; g < G; g++) {
        uint16_t range = kvo_f2h(gmax[g] - gmin[g]);                 /* (max_ - min_) in fp16        */
        uint16_t scale = kvo_f2h(kvo_h2f(range) * eb);               /* * quant_scale_rel (f32 scalar)*/
        uint16_t mq = kvo_f2h(gmin[g] / kvo_h2f(scale));             /* min_ / quant_scale            */
        uint16_t mi = kvo_f2h(rintf(kvo_h2f(mq)));                   /* .round_()  (half-to-even)     */
        scale_f16[g] = scale;
        min_f16[g] = mi;
        if (min_i8) min_i8[g] = (int8_t)(int32_t)kvo_h2f(mi);        /* kvcomp_encode.py:97           */
    }
    idx = 0;
    for (int64_t nb = 0; nb < NB; nb++)
      for (int64_t bs = 0; bs < BS; bs++)
        for (int64_t b = 0; b < B; b++)
          for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++, idx++) {
                int64_t g = kvo_group_index(nb, bs, b, h, d, BS, B, H, D, mask);
                float sc = kvo_h2f(scale_f16[g]);
                uint16_t q = kvo_f2h(kvo_h2f(x[idx]) / sc);          /* tensor / quant_scale          */
                q = kvo_f2h(rintf(kvo_h2f(q)));                      /* .round_()                     */
                uint16_t s = kvo_f2h(kvo_h2f(q) - kvo_h2f(min_f16[g]));   /* quant_ints - min_ints    */
                if (sym_f16) sym_f16[idx] = s;
                if (sym_u8) sym_u8[idx] = (uint8_t)(int32_t)kvo_h2f(s);   /* kvcomp_encode.py:98      */
            }
    free(gmin);
    free(gmax);
    return 0;
}

/* Q2  dequantizer: (sym + min_i) * scale.  models/cache/kvcomp_encode.py:146,161; utils/compute.py:130.
 * uint8 + int8 promotes to int16 (exact); int16 * fp16 -> RN16(f32(int) * f32(scale)).           */
void kvo_dequant(const uint8_t *sym, const int8_t *min_i8, const uint16_t *scale_f16,
                 int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int mask, uint16_t *out_f16)
{
    int64_t idx = 0;
    for (int64_t nb = 0; nb < NB; nb++)
      for (int64_t bs = 0; bs < BS; bs++)
        for (int64_t b = 0; b < B; b++)
          for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++, idx++) {
                int64_t g = kvo_group_index(nb, bs, b, h, d, BS, B, H, D, mask);
                int v = (int)sym[idx] + (int)min_i8[g];
                out_f16[idx] = kvo_f2h((float)v * kvo_h2f(scale_f16[g]));
            }
}

/* Q3  error-bound invariant |x - xhat| < 0.53*scale.  src/compute.cpp:60-69.
 * Evaluated like the reference would: fp16 subtract, fp16 abs, fp16 product, fp16 compare.
 * Returns the number of violating elements.                                                   */
int64_t kvo_check_error_bound(const uint16_t *x, const uint16_t *xhat, const uint16_t *scale_f16,
                              int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int mask)
{
    int64_t idx = 0, bad = 0;
    for (int64_t nb = 0; nb < NB; nb++)
      for (int64_t bs = 0; bs < BS; bs++)
        for (int64_t b = 0; b < B; b++)
          for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++, idx++) {
                int64_t g = kvo_group_index(nb, bs, b, h, d, BS, B, H, D, mask);
                float err = fabsf(kvo_h2f(kvo_f2h(kvo_h2f(x[idx]) - kvo_h2f(xhat[idx]))));
                float lim = kvo_h2f(kvo_f2h(kvo_h2f(scale_f16[g]) * 0.53f));
                if (!(err < lim)) bad++;
            }
    return bad;
}

/* C1  how many whole blocks leave the uncompressed tail.  utils/compute.py:59-72 (and :44-57). */
int64_t kvo_blocks_to_compress(int64_t len, int64_t block_size, int64_t recent_size)
{
    int64_t res = len % block_size;
    int64_t num = len + block_size - res - recent_size;
    /* Python floor division */
    int64_t q = num / block_size;
    if ((num % block_size != 0) && ((num < 0) != (block_size < 0))) q--;
    return q;
}

/* ------------------------------------------------------------------------------------------ */
/* H1/H2  tie-exact Huffman construction.                                                      */
/*   src/huffman.cpp:34-96  (std::priority_queue on frequency only, leaves pushed in ascending */
/*                           symbol order, first pop = left = '0')                             */
/*   utils/huffman.py:46-81 (heapq with __lt__ on freq only, same merge rule)                  */
/* Both containers are the same array heap: push = append + sift up while child < parent;     */
/* pop = move the hole from the root to a leaf always taking the smaller child (the right one  */
/* on ties), drop the former last element there and sift it up.  The heap is written out here  */
/* so the result does not depend on any library.                                               */
/*   h2_single = 0: a lone symbol gets the empty code, length 0  (huffman.cpp:60-71)           */
/*   h2_single = 1: a lone symbol gets '0', length 1             (utils/huffman.py:42-44)      */
/* Returns the number of distinct symbols, or -1 if a code would exceed 32 bits (the           */
/* reference stores codes in a u32, include/huffman.h:13-16).                                  */
/* ------------------------------------------------------------------------------------------ */
typedef struct { int64_t f; int left, right, sym; } kvo_node;

static void kvo_heap_push(int *heap, int *n, const kvo_node *nodes, int x)
{
    int pos = (*n)++;
    while (pos > 0) {
        int par = (pos - 1) >> 1;
        if (nodes[x].f < nodes[heap[par]].f) { heap[pos] = heap[par]; pos = par; }
        else break;
    }
    heap[pos] = x;
}

static int kvo_heap_pop(int *heap, int *n, const kvo_node *nodes)
{
    int last = heap[--(*n)];
    if (*n == 0) return last;
    int top = heap[0], pos = 0, child = 1, cnt = *n;
    while (child < cnt) {
        int right = child + 1;
        if (right < cnt && !(nodes[heap[child]].f < nodes[heap[right]].f)) child = right;
        heap[pos] = heap[child];
        pos = child;
        child = 2 * pos + 1;
    }
    while (pos > 0) {
        int par = (pos - 1) >> 1;
        if (nodes[last].f < nodes[heap[par]].f) { heap[pos] = heap[par]; pos = par; }
        else break;
    }
    heap[pos] = last;
    return top;
}

int kvo_huffman_build(const int64_t *counts, int nsymbols, int h2_single, uint32_t *code, uint32_t *length)
{
    kvo_node *nodes = (kvo_node *)malloc(sizeof(kvo_node) * (size_t)(2 * nsymbols + 2));
    int *heap = (int *)malloc(sizeof(int) * (size_t)(nsymbols + 2));
    int *stack = (int *)malloc(sizeof(int) * (size_t)(2 * nsymbols + 2));
    uint64_t *scode = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)(2 * nsymbols + 2));
    int *slen = (int *)malloc(sizeof(int) * (size_t)(2 * nsymbols + 2));
    int nn = 0, hn = 0, distinct = 0, rc = 0;
    for (int s = 0; s < nsymbols; s++) { code[s] = 0; length[s] = 0; }
    for (int s = 0; s < nsymbols; s++) {
        if (counts[s] > 0) {
            nodes[nn].f = counts[s]; nodes[nn].left = nodes[nn].right = -1; nodes[nn].sym = s;
            kvo_heap_push(heap, &hn, nodes, nn);
            nn++; distinct++;
        }
    }
    if (distinct == 0) goto done;
    if (distinct == 1) {
        int s = nodes[0].sym;
        code[s] = 0; length[s] = h2_single ? 1u : 0u;
        goto done;
    }
    while (hn > 1) {
        int a = kvo_heap_pop(heap, &hn, nodes);
        int b = kvo_heap_pop(heap, &hn, nodes);
        nodes[nn].f = nodes[a].f + nodes[b].f; nodes[nn].left = a; nodes[nn].right = b; nodes[nn].sym = -1;
        kvo_heap_push(heap, &hn, nodes, nn);
        nn++;
    }
    {
        int sp = 0;
        stack[sp] = heap[0]; scode[sp] = 0; slen[sp] = 0; sp++;
        while (sp > 0) {
            sp--;
            int nd = stack[sp]; uint64_t c = scode[sp]; int l = slen[sp];
            if (nodes[nd].left < 0) {
                if (l > 32) { rc = -1; goto done; }
                code[nodes[nd].sym] = (uint32_t)c; length[nodes[nd].sym] = (uint32_t)l;
            } else {
                if (l >= 63) { rc = -1; goto done; }
                stack[sp] = nodes[nd].right; scode[sp] = (c << 1) | 1u; slen[sp] = l + 1; sp++;
                stack[sp] = nodes[nd].left;  scode[sp] = (c << 1);      slen[sp] = l + 1; sp++;
            }
        }
    }
done:
    free(nodes); free(heap); free(stack); free(scode); free(slen);
    return rc < 0 ? rc : distinct;
}

/* T1  encode table.  include/huffman.h:13-16, src/huffman.cpp:111-131,166-187.
 * (max_sym - min_sym + 1) entries of {u32 code; u32 length}, little-endian, indexed by
 * symbol - min_sym; symbols that never occur are all-zero entries.  Returns the byte count
 * written to `table` (0 if there is no symbol) and the shift (= min symbol) through *shift.   */
int64_t kvo_encode_table(const uint32_t *code, const uint32_t *length, const int64_t *counts, int nsymbols,
                         uint8_t *table, int *shift)
{
    int mn = -1, mx = -1;
    for (int s = 0; s < nsymbols; s++) if (counts[s] > 0) { if (mn < 0) mn = s; mx = s; }
    if (mn < 0) { *shift = 255; return 0; }
    *shift = mn;
    int64_t n = mx - mn + 1;
    memset(table, 0, (size_t)n * 8);
    for (int s = mn; s <= mx; s++) {
        if (counts[s] <= 0) continue;
        uint32_t c = code[s], l = length[s];
        uint8_t *p = table + (size_t)(s - mn) * 8;
        p[0] = (uint8_t)c; p[1] = (uint8_t)(c >> 8); p[2] = (uint8_t)(c >> 16); p[3] = (uint8_t)(c >> 24);
        p[4] = (uint8_t)l; p[5] = (uint8_t)(l >> 8); p[6] = (uint8_t)(l >> 16); p[7] = (uint8_t)(l >> 24);
    }
    return n * 8;
}

/* T2  decode tree array.  include/huffman.h:18-22, src/huffman.cpp:229-252.
 * 3-byte nodes {u8 is_leaf; i8 a; i8 b}; nodes 0 and 1 are the root's children for bit 0 / 1;
 * symbols are inserted in ascending order and nodes appended on demand; a leaf stores the symbol
 * in both slots.  Child indices and symbols are stored as int8 exactly like the reference, so
 * more than 127 nodes (64 symbols) or symbols above 127 wrap: the function still writes what the
 * reference would and returns -2 to flag that the tree is unusable.  A length-0 code (lone
 * symbol) indexes node -1 in the reference (undefined): returns -3 and writes the two empty
 * root children only.  Otherwise returns the byte count.                                      */
int64_t kvo_decode_tree(const uint32_t *code, const uint32_t *length, const int64_t *counts, int nsymbols,
                        uint8_t *tree, int64_t tree_cap_bytes)
{
    int64_t nn = 2, rc = 0;
    if (tree_cap_bytes < 6) return -1;
    for (int k = 0; k < 2; k++) { tree[3 * k] = 0; tree[3 * k + 1] = 0xff; tree[3 * k + 2] = 0xff; }
    for (int s = 0; s < nsymbols; s++) {
        if (counts[s] <= 0) continue;
        if (length[s] == 0) { rc = -3; continue; }
        int idx = -1, last = -1;
        for (uint32_t i = 0; i < length[s]; i++) {
            int bit = (int)((code[s] >> (length[s] - 1 - i)) & 1u);
            idx = (idx == -1) ? bit : (int)(int8_t)tree[3 * idx + 1 + bit];
            if (idx == -1) {
                if ((nn + 1) * 3 > tree_cap_bytes) return -1;
                tree[3 * nn] = 0; tree[3 * nn + 1] = 0xff; tree[3 * nn + 2] = 0xff;
                tree[3 * last + 1 + bit] = (uint8_t)(int8_t)nn;
                if (nn > 127) rc = -2;
                idx = (int)nn;
                nn++;
            } else if (idx < 0) {
                return -2;   /* a wrapped (negative, not -1) child index: the reference would read out of bounds */
            }
            last = idx;
        }
        tree[3 * idx] = 1;
        tree[3 * idx + 1] = (uint8_t)(int8_t)s;
        tree[3 * idx + 2] = (uint8_t)(int8_t)s;
        if (s > 127) rc = -2;
    }
    return rc < 0 ? rc : nn * 3;
}

/* H2  whole-tensor bitstream of utils/huffman.py:15-95: codes of the flattened symbols
 * concatenated; one output byte (0/1) per bit, like the torch.bool tensor it returns.
 * Returns the bit count (or -1 if `cap` is too small).                                        */
int64_t kvo_huffman_bits(const uint8_t *sym, int64_t n, const uint32_t *code, const uint32_t *length,
                         uint8_t *bits, int64_t cap)
{
    int64_t nb = 0;
    for (int64_t i = 0; i < n; i++) {
        uint32_t c = code[sym[i]], l = length[sym[i]];
        if (nb + l > cap) return -1;
        for (uint32_t k = 0; k < l; k++) bits[nb++] = (uint8_t)((c >> (l - 1 - k)) & 1u);
    }
    return nb;
}

/* ------------------------------------------------------------------------------------------ */
/* E1-E3  tile encoder.  src/kernels.cu:181-235 (entropy_encode), :419-596 (K and V tile       */
/* kernels), :893-917 (sizes); include/kernels.h:25-42 (block_info, thread_info).              */
/*                                                                                             */
/* Input symbols u8 [NB, BS, B, H, D] contiguous; stride = B*H*D bytes per token.              */
/*   K: tile = 64 tokens x vec_len flat channels; lane t encodes token 64*row+t, channels      */
/*      vec_len*col .. +vec_len-1 ascending.  (reference: vec_len = 128)                       */
/*   V: tile = vec_len tokens x 64 flat channels; lane t encodes channel 64*col+t, tokens      */
/*      vec_len*row .. ascending.               (reference: vec_len = 128)                     */
/* A lane's stream is its codes MSB-first, zero padded to a whole byte; the tile payload is    */
/* the 64 streams back to back.  thread_info = end_byte*8 + pad (u16, wraps like the           */
/* reference's static_cast).  block_info = {u32 offset; u16 byte_num; 2 pad bytes}.            */
/* Tiles are laid out in tile order (the reference uses atomic arrival order, kernels.cu:474;  */
/* offsets are therefore compared per tile, never across tiles).                               */
/* The encode table is indexed by the raw symbol (kernels.cu:197), i.e. shift must be 0.       */
/* Returns total payload bytes, or -1 on capacity overflow, -2 if a symbol has no code.        */
/* ------------------------------------------------------------------------------------------ */
static inline uint32_t kvo_rd32(const uint8_t *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

int64_t kvo_tile_count(int64_t tokens, int64_t stride, int is_k, int vec_len)
{
    if (is_k) return (tokens / KVO_VEC_PER_TILE) * (stride / vec_len);
    return (tokens / vec_len) * (stride / KVO_VEC_PER_TILE);
}

int64_t kvo_encode_tiles(const uint8_t *sym, int64_t tokens, int64_t stride, int is_k, int vec_len,
                         const uint8_t *table, int64_t table_entries, uint32_t base_global_offset,
                         uint8_t *payload, int64_t payload_cap, uint8_t *block_infos, uint8_t *thread_infos)
{
    int64_t tiles = kvo_tile_count(tokens, stride, is_k, vec_len);
    int64_t cols = is_k ? stride / vec_len : stride / KVO_VEC_PER_TILE;
    int64_t total = 0;
    for (int64_t tau = 0; tau < tiles; tau++) {
        int64_t row = tau / cols, col = tau % cols;
        int64_t tile_start = total;
        for (int t = 0; t < KVO_VEC_PER_TILE; t++) {
            uint64_t acc = 0; int nacc = 0; int64_t bits = 0, start = total;
            for (int i = 0; i < vec_len; i++) {
                int64_t at = is_k ? (row * KVO_VEC_PER_TILE + t) * stride + col * vec_len + i
                                  : (row * vec_len + i) * stride + col * KVO_VEC_PER_TILE + t;
                uint8_t s = sym[at];
                if (s >= table_entries) return -2;
                uint32_t c = kvo_rd32(table + 8 * (size_t)s), l = kvo_rd32(table + 8 * (size_t)s + 4);
                if (l == 0 || l > 32) return -2;
                acc = (acc << l) | c; nacc += (int)l; bits += l;
                while (nacc >= 8) {
                    if (total >= payload_cap) return -1;
                    payload[total++] = (uint8_t)(acc >> (nacc - 8));
                    nacc -= 8;
                }
                acc &= (nacc ? ((1ull << nacc) - 1ull) : 0ull);
            }
            if (nacc > 0) {
                if (total >= payload_cap) return -1;
                payload[total++] = (uint8_t)(acc << (8 - nacc));
            }
            int64_t bytes = total - start, end = total - tile_start;
            uint16_t ti = (uint16_t)((end << 3) + (bytes << 3) - bits);
            size_t v = (size_t)(tau * KVO_VEC_PER_TILE + t);
            thread_infos[2 * v] = (uint8_t)ti; thread_infos[2 * v + 1] = (uint8_t)(ti >> 8);
        }
        uint32_t off = (uint32_t)tile_start + base_global_offset;
        uint16_t bn = (uint16_t)(total - tile_start);
        uint8_t *bi = block_infos + 8 * (size_t)tau;
        bi[0] = (uint8_t)off; bi[1] = (uint8_t)(off >> 8); bi[2] = (uint8_t)(off >> 16); bi[3] = (uint8_t)(off >> 24);
        bi[4] = (uint8_t)bn; bi[5] = (uint8_t)(bn >> 8); bi[6] = 0; bi[7] = 0;
    }
    return total;
}

/* ------------------------------------------------------------------------------------------ */
/* D1/D2  tile decoder: bit-serial tree walk.  src/kernels.cu:237-291 (entropy_decode),        */
/* :598-719 (lane start = previous lane's end byte, bit budget = bytes*8 - pad; transposed     */
/* store back into [NB, BS, B, H, D]).  `tree` is the T2 array.  Each lane must yield exactly  */
/* vec_len symbols; returns 0, or -(1 + first failing vector index).                           */
/* ------------------------------------------------------------------------------------------ */
static int kvo_walk(const uint8_t *tree, int64_t tree_nodes, const uint8_t *in, int64_t nbits,
                    uint8_t *out, int vec_len)
{
    int idx = -1, n = 0;
    for (int64_t k = 0; k < nbits; k++) {
        int bit = (in[k >> 3] >> (7 - (k & 7))) & 1;
        idx = (idx == -1) ? bit : (int)(int8_t)tree[3 * idx + 1 + bit];
        if (idx < 0 || idx >= tree_nodes) return -1;
        if (tree[3 * idx]) {
            if (n >= vec_len) return -1;
            out[n++] = tree[3 * idx + 1];
            idx = -1;
        }
    }
    return n;
}

int64_t kvo_decode_tiles(const uint8_t *encoded, const uint8_t *block_infos, const uint8_t *thread_infos,
                         const uint8_t *tree, int64_t tree_bytes, int64_t tokens, int64_t stride,
                         int is_k, int vec_len, uint8_t *out)
{
    int64_t tiles = kvo_tile_count(tokens, stride, is_k, vec_len);
    int64_t cols = is_k ? stride / vec_len : stride / KVO_VEC_PER_TILE;
    uint8_t tmp[256];
    if (vec_len > 256) return -1;
    for (int64_t tau = 0; tau < tiles; tau++) {
        int64_t row = tau / cols, col = tau % cols;
        const uint8_t *bi = block_infos + 8 * (size_t)tau;
        uint32_t off = kvo_rd32(bi);
        for (int t = 0; t < KVO_VEC_PER_TILE; t++) {
            size_t v = (size_t)(tau * KVO_VEC_PER_TILE + t);
            uint16_t ti = (uint16_t)(thread_infos[2 * v] | (thread_infos[2 * v + 1] << 8));
            uint16_t prev = t ? (uint16_t)(thread_infos[2 * v - 2] | (thread_infos[2 * v - 1] << 8)) : 0;
            int64_t start = t ? (prev >> 3) : 0;
            int64_t nbits = (((int64_t)(ti >> 3) - start) << 3) - (ti & 7);
            int n = kvo_walk(tree, tree_bytes / 3, encoded + off + start, nbits, tmp, vec_len);
            if (n != vec_len) return -(1 + (int64_t)v);
            for (int i = 0; i < vec_len; i++) {
                int64_t at = is_k ? (row * KVO_VEC_PER_TILE + t) * stride + col * vec_len + i
                                  : (row * vec_len + i) * stride + col * KVO_VEC_PER_TILE + t;
                out[at] = tmp[i];
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* F1  decode -> dequantize -> q.K^T.  src/kernels.cu:293-348,721-776 (operand layout) with    */
/* the dequantizer of Q2; the sum is carried in double, so it is the exact value that both the */
/* reference's fp16 chain and this build's fp32 chain approximate.                             */
/*   sym   u8 [T, B, H, D]  (already decoded),  q fp16 [B, Hq, D],  score f64 [B, Hq, T]       */
/*   K (min, scale) group layout given by mask as in kvo_quant; query head hq reads KV head    */
/*   hq / (Hq / H).                                                                            */
/* ------------------------------------------------------------------------------------------ */
void kvo_fused_k(const uint8_t *sym, const int8_t *min_i8, const uint16_t *scale_f16, int mask,
                 int64_t T, int64_t BS, int64_t B, int64_t H, int64_t D,
                 const uint16_t *q, int64_t Hq, double *score)
{
    int64_t rep = Hq / H;
    for (int64_t b = 0; b < B; b++)
      for (int64_t hq = 0; hq < Hq; hq++) {
        int64_t h = hq / rep;
        for (int64_t t = 0; t < T; t++) {
            double acc = 0.0;
            for (int64_t d = 0; d < D; d++) {
                int64_t g = kvo_group_index(t / BS, t % BS, b, h, d, BS, B, H, D, mask);
                int v = (int)sym[((t * B + b) * H + h) * D + d] + (int)min_i8[g];
                float k = kvo_h2f(kvo_f2h((float)v * kvo_h2f(scale_f16[g])));
                acc += (double)k * (double)kvo_h2f(q[(b * Hq + hq) * D + d]);
            }
            score[(b * Hq + hq) * T + t] = acc;
        }
      }
}

/* F2  decode -> dequantize -> p.V.  src/kernels.cu:350-407,778-861 + the caller's sum over
 * 128-token groups (models/cache/kvcomp_encode.py:275).  p fp16 [B, Hq, T], out f64 [B, Hq, D]. */
void kvo_fused_v(const uint8_t *sym, const int8_t *min_i8, const uint16_t *scale_f16, int mask,
                 int64_t T, int64_t BS, int64_t B, int64_t H, int64_t D,
                 const uint16_t *p, int64_t Hq, double *out)
{
    int64_t rep = Hq / H;
    for (int64_t b = 0; b < B; b++)
      for (int64_t hq = 0; hq < Hq; hq++) {
        int64_t h = hq / rep;
        for (int64_t d = 0; d < D; d++) {
            double acc = 0.0;
            for (int64_t t = 0; t < T; t++) {
                int64_t g = kvo_group_index(t / BS, t % BS, b, h, d, BS, B, H, D, mask);
                int v = (int)sym[((t * B + b) * H + h) * D + d] + (int)min_i8[g];
                float val = kvo_h2f(kvo_f2h((float)v * kvo_h2f(scale_f16[g])));
                acc += (double)val * (double)kvo_h2f(p[(b * Hq + hq) * T + t]);
            }
            out[(b * Hq + hq) * D + d] = acc;
        }
      }
}

/* ------------------------------------------------------------------------------------------ */
/* CPU baseline leg: the reference's fused K path end to end on the host, as its kernel does    */
/* it per lane -- bit-serial tree walk straight out of the payload, fp16 dequantize, dot with   */
/* q -- (src/kernels.cu:293-348,721-776), with an fp32 accumulator.  mask 0xF: one (min, scale)  */
/* per 64-token block (kernels.cu:771-772); mask 0x1: one per (block, b, h, channel).           */
/* score fp32 [B*H, T].  Returns 0 or a negative vector index on a malformed stream.            */
/* ------------------------------------------------------------------------------------------ */
int64_t kvo_fused_k_from_stream(const uint8_t *encoded, const uint8_t *block_infos, const uint8_t *thread_infos,
                                const uint8_t *tree, int64_t tree_bytes,
                                const int8_t *min_i8, const uint16_t *scale_f16, int mask,
                                const uint16_t *q, int64_t tokens, int64_t stride, int vec_len, float *score)
{
    int64_t cols = stride / vec_len, rows = tokens / KVO_VEC_PER_TILE, tiles = rows * cols;
    int64_t tree_nodes = tree_bytes / 3, rc = 0;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t tau = 0; tau < tiles; tau++) {
        int64_t row = tau / cols, col = tau % cols;
        uint32_t off = kvo_rd32(block_infos + 8 * (size_t)tau);
        const int per_channel = (mask == 0x1);
        const int8_t *mnp = per_channel ? min_i8 + tau * vec_len : min_i8 + row;
        const uint16_t *scp = per_channel ? scale_f16 + tau * vec_len : scale_f16 + row;
        for (int t = 0; t < KVO_VEC_PER_TILE; t++) {
            size_t v = (size_t)(tau * KVO_VEC_PER_TILE + t);
            uint16_t ti = (uint16_t)(thread_infos[2 * v] | (thread_infos[2 * v + 1] << 8));
            uint16_t prev = t ? (uint16_t)(thread_infos[2 * v - 2] | (thread_infos[2 * v - 1] << 8)) : 0;
            int64_t start = t ? (prev >> 3) : 0;
            int64_t nbits = (((int64_t)(ti >> 3) - start) << 3) - (ti & 7);
            const uint8_t *in = encoded + off + start;
            int idx = -1, n = 0;
            float acc = 0.f;
            for (int64_t k = 0; k < nbits; k++) {
                int bit = (in[k >> 3] >> (7 - (k & 7))) & 1;
                idx = (idx == -1) ? bit : (int)(int8_t)tree[3 * idx + 1 + bit];
                if (idx < 0 || idx >= tree_nodes) { rc = -(1 + (int64_t)v); break; }
                if (tree[3 * idx]) {
                    if (n < vec_len) {
                        int mn = per_channel ? mnp[n] : mnp[0];
                        float sc = kvo_h2f(per_channel ? scp[n] : scp[0]);
                        float kv = kvo_h2f(kvo_f2h((float)((int)tree[3 * idx + 1] + mn) * sc));
                        acc += kv * kvo_h2f(q[col * vec_len + n]);
                    }
                    n++;
                    idx = -1;
                }
            }
            score[col * tokens + row * KVO_VEC_PER_TILE + t] = acc;
        }
    }
    return rc;
}

/* Thread count of the CPU baseline leg (OpenMP over tiles); returns the count in effect. */
int kvo_set_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}
