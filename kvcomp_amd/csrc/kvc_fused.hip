// kvc_fused.hip -- Huffman decode fused with the two matvecs of decode attention: decoded symbols go
// from the LDS lookup straight into an fp32 FMA and never reach HBM.
//
//   kvc_fused_kernel<REP, true>   <- huffman_decode_and_mat_vec_mul   (kvcomp_cuda_extension/src/kernels.cu:721-776)
//   kvc_fused_kernel<REP, false>  <- v_huffman_decode_and_mat_vec_mul (kernels.cu:778-861)
//
// One wave64 per tile, lane t owns stream t (K: a token, V: a channel), exactly the reference's work split.
// Every lane decodes one symbol per step, so step i means "channel i" (K) or "token i of the 128-token
// group" (V) for the whole wave and the other FMA operand is wave-uniform:
//   K: score  = sum_i (sym_i + min_i) scale_i q_i = sum_i sym_i q'_i + sum_i min_i q'_i,  q'_i = scale_i q_i
//   V: out_d  = sum_t (sym_t + min_t) scale_t p_t = sum_t sym_t w_t  + sum_t min_t w_t,   w_t  = scale_t p_t
// q' / w are computed once per tile into two VGPRs per query head (lane l holds elements l and l + 64) and
// reach the FMA through v_readlane.  REP query heads share one KV head (grouped-query attention): the tile
// is decoded once and feeds REP accumulators.
//
// Inner loop (the "fast" path, codes no longer than the table index):
//   window  32 stream bits, rotated so that the next `lbits` bits sit at bits [lbits+1 : 2] -- masking gives
//           the byte offset of the table entry directly
//   entry   fp32 bit pattern of the symbol with (32 - len) in the 5 lowest mantissa bits: it is the FMA
//           operand as it stands, and as a shift count it rotates the window left by len (v_alignbit)
//   refill  every 4 (or 8) symbols the window is re-read from the staged payload at the lane's bit position;
//           the entries are summed so the low byte of the sum gives the bits consumed
// A 32-bit window always suffices for 8 symbols of <= 4 bits or 4 symbols of <= 8 bits.  With longer codes
// 4 symbols can, very rarely, need more than 32 bits: lanes note the largest consumption they saw, and if
// any lane went over, the wave decodes that tile again on the slow path.
//
// Slow path (codebooks with codes longer than the table index, tiles larger than the staging area, or
// the rare overflow above): one symbol per refill, generic table read from global memory, payload read
// from LDS or -- for an oversized tile -- from global memory.
#include "kvc_tile.h"

struct KvcFusedArgs {
    KvcStreamArgs s;
    const int8_t *min_i8;
    const __half *scale;
    int quant_mask;
    const __half *x;     // K: q [batch, q_heads, head_dim];  V: p [batch, q_heads, tokens]
    void *out;           // K: scores [batch, q_heads, tokens]; V: partial [tokens/128, batch, q_heads, head_dim]
    int out_f32;         // 0: fp16 (reference layout), 1: fp32
    int64_t tokens;
    int batch, kv_heads, q_heads, head_dim;
    int stage_words;     // LDS words per wave for the staged payload
};

constexpr int KVC_STAGE_LEAD_WORDS = 4;   // the payload is staged from word 4 on, so bit positions are never 0

// -- staging ----------------------------------------------------------------------------------------
struct KvcTile {
    const uint32_t *gwords;   // 16-byte aligned global address of the chunk that holds the first payload byte
    uint32_t nwords;          // whole words from gwords that contain payload bytes
    uint32_t pos;             // this lane's first stream bit, counted from gwords (global) / from the stage base + lead
    bool fits;                // payload is in LDS
};

__device__ __forceinline__ KvcTile kvc_stage_tile_lds(const KvcStreamArgs &a, int64_t tile, uint32_t *stage,
                                                      int stage_words, int lane)
{
    const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.block_infos + 8 * tile);
    uint32_t off = bi[0];
    uint32_t bn = bi[1] & 0xffffu;
    if (bn > (uint32_t)KVC_MAX_TILE_BYTES) bn = KVC_MAX_TILE_BYTES;
    if ((int64_t)off >= a.enc_bytes) bn = 0;
    else if ((int64_t)off + bn > a.enc_bytes) bn = (uint32_t)(a.enc_bytes - off);
    const uintptr_t src = reinterpret_cast<uintptr_t>(a.enc) + off;
    const uintptr_t base = src & ~(uintptr_t)15;
    const uint32_t head = (uint32_t)(src - base);
    const uint32_t nchunks = bn ? (head + bn + 15u) >> 4 : 0u;
    KvcTile t;
    t.gwords = reinterpret_cast<const uint32_t *>(base);
    t.nwords = (head + bn + 3u) >> 2;
    // lead words + chunks + two look-ahead words must fit
    t.fits = (int)(KVC_STAGE_LEAD_WORDS + 4 * nchunks + 2) <= stage_words;
    if (t.fits) {
        const uint4 *g = reinterpret_cast<const uint4 *>(base);
        uint4 *s = reinterpret_cast<uint4 *>(stage + KVC_STAGE_LEAD_WORDS);
        for (uint32_t c = lane; c < nchunks; c += KVC_WAVE) {
            uint4 v = g[c];
            v.x = kvc_bswap(v.x);
            v.y = kvc_bswap(v.y);
            v.z = kvc_bswap(v.z);
            v.w = kvc_bswap(v.w);
            s[c] = v;
        }
    }
    uint32_t start = lane ? (uint32_t)(a.thread_infos[tile * KVC_WAVE + lane - 1] >> 3) : 0u;
    if (start > bn) start = bn;
    t.pos = (head + start) * 8u;
    return t;
}

// -- slow path ----------------------------------------------------------------------------------------
// One symbol per refill; table and long-code list in global memory; words from LDS (already big-endian)
// or from global memory (raw, swapped on the fly, bounds-checked word by word).
// Returns sum_i sym_i * ops[i * REP + r] for each query head r (ops: this lane's operand table in LDS).
template <int REP>
struct KvcVec {
    float v[REP];
};

template <int REP, bool GSRC>
__device__ __noinline__ KvcVec<REP> kvc_slow_tile(const uint32_t *words, uint32_t nwords, uint32_t pos,
                                                  const uint32_t *__restrict__ lut_g, int n, const float *ops)
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
        if (wi < nwords) w0 = GSRC ? kvc_bswap(words[wi]) : words[wi];
        if (wi + 1 < nwords) w1 = GSRC ? kvc_bswap(words[wi + 1]) : words[wi + 1];
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
#pragma unroll
        for (int r = 0; r < REP; r++) acc.v[r] = fmaf(f, ops[i * REP + r], acc.v[r]);
        pos += len;
    }
    return acc;
}

// -- fast path ----------------------------------------------------------------------------------------
// n symbols (a multiple of G) starting at bit t + 1 of the staged words; acc[r] += sym_i * ops[i * REP + r].
// `ops` is this lane's view of the wave's operand table in LDS: the same address in every lane (a broadcast
// read) except in V tiles that straddle two heads, where the lanes of the second head point at its table.
// Returns through `t` the new position and through `worst` the largest number of bits a group consumed.
template <int G, bool CHECK, int REP>
__device__ __forceinline__ void kvc_fast_dot(const uint32_t *stage, uint32_t last_word, uint32_t &t,
                                             const char *fentry_bytes, uint32_t mask4, uint32_t rot, int n,
                                             const float *ops, float (&acc)[REP], uint32_t &worst)
{
#pragma unroll 2
    for (int i = 0; i < n; i += G) {
        uint32_t a = t >> 5;
        a = a < last_word ? a : last_word;
        const uint32_t w0 = stage[a], w1 = stage[a + 1];
        float op[G * REP];
#pragma unroll
        for (int k = 0; k < G * REP; k += 4) {
            const float4 v = *reinterpret_cast<const float4 *>(ops + i * REP + k);
            op[k] = v.x;
            if (k + 1 < G * REP) op[k + 1] = v.y;
            if (k + 2 < G * REP) op[k + 2] = v.z;
            if (k + 3 < G * REP) op[k + 3] = v.w;
        }
        const uint32_t win = __builtin_amdgcn_alignbit(w0, w1, ~t);   // 32 bits from stream bit t + 1
        uint32_t R = __builtin_amdgcn_alignbit(win, win, rot);        // next lbits bits -> [lbits+1 : 2]
        uint32_t es = 0;
#pragma unroll
        for (int g = 0; g < G; g++) {
            const uint32_t e = *reinterpret_cast<const uint32_t *>(fentry_bytes + (R & mask4));
            R = __builtin_amdgcn_alignbit(R, R, e);                   // rotate left by len
            es += e;
            const float f = __uint_as_float(e);
#pragma unroll
            for (int r = 0; r < REP; r++) acc[r] = fmaf(f, op[g * REP + r], acc[r]);
        }
        const uint32_t used = 32u * G - (es & 0xffu);
        if (CHECK) worst = used > worst ? used : worst;
        t += used;
    }
}

// Operand table of one wave: [head slot (1 or 2)][128 elements][REP] floats.
template <int REP>
__host__ __device__ constexpr int kvc_op_words(int slots) { return slots * 128 * REP; }

template <int REP, bool IS_K>
__global__ void __launch_bounds__(KVC_WG) kvc_fused_kernel(KvcFusedArgs a)
{
    __shared__ __align__(16) uint32_t s_fentry[KVC_LUT_ENTRY_WORDS];   // static: its LDS offset folds into ds_read
    extern __shared__ __align__(16) uint32_t smem[];                   // per wave: operand table, then staged payload
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int D = a.head_dim;
    const int slots = (!IS_K && (D % KVC_WAVE) != 0) ? 2 : 1;          // V tiles may straddle two heads
    const int per_wave = kvc_op_words<REP>(slots) + a.stage_words;
    float *ops = reinterpret_cast<float *>(smem + wave * per_wave);
    uint32_t *stage = smem + wave * per_wave + kvc_op_words<REP>(slots);
    const int row = blockIdx.y;
    const int64_t cb = a.s.rows_per_codebook ? row / a.s.rows_per_codebook : 0;
    const uint32_t *__restrict__ lut_g = a.s.luts + cb * KVC_LUT_WORDS;
    const uint32_t lbits = lut_g[0], lmax = lut_g[1], nlong = lut_g[2];
    const bool fast_book = nlong == 0 && lbits <= (uint32_t)KVC_LUT_MAX_BITS;
    if (fast_book)
        for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) s_fentry[i] = lut_g[KVC_LUT_FENTRY_OFFSET + i];
    if (lane < KVC_STAGE_LEAD_WORDS) stage[lane] = 0;
    __syncthreads();
    const uint32_t mask4 = ((1u << lbits) - 1u) << 2;
    const uint32_t rot = 30u - lbits;                                  // (32 - lbits) - 2
    const uint32_t last_word = (uint32_t)a.stage_words - 2u;
    const int n = IS_K ? D : KVC_V_TOKENS;                             // symbols per lane stream

    for (int it = 0; it < a.s.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.s.tiles_per_wave + it;
        const bool active = col < a.s.cols;
        const int64_t tile = (int64_t)row * a.s.cols + col;
        KvcTile tl;
        tl.fits = false;
        float bias[REP];
        int64_t out_base = 0, out_step = 0;
        const float *my_ops = ops;
        if (active) {
            tl = kvc_stage_tile_lds(a.s, tile, stage, a.stage_words, lane);
            // ---- per-tile operand table: element i of head slot s, query head r at ops[(s*128 + i)*REP + r]
            if (IS_K) {
                const int b = col / a.kv_heads, h = col - b * a.kv_heads;
#pragma unroll
                for (int r = 0; r < REP; r++) bias[r] = 0.f;
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    const int i = lane + 64 * half;
                    float sc = 0.f, mn = 0.f;
                    if (i < D) {
                        if (a.quant_mask == KVC_MASK_CHANNEL) {
                            sc = __half2float(a.scale[tile * D + i]);
                            mn = (float)a.min_i8[tile * D + i];
                        } else {   // KVC_MASK_K_BLOCK: one pair per 64-token block (kernels.cu:771-772)
                            sc = __half2float(a.scale[row]);
                            mn = (float)a.min_i8[row];
                        }
                    }
#pragma unroll
                    for (int r = 0; r < REP; r++) {
                        const __half *qp = a.x + ((int64_t)b * a.q_heads + h * REP + r) * D;
                        const float v = i < D ? sc * __half2float(qp[i]) : 0.f;
                        ops[i * REP + r] = v;
                        bias[r] += mn * v;
                    }
                }
                out_base = ((int64_t)b * a.q_heads + h * REP) * a.tokens + (int64_t)row * KVC_WAVE + lane;
                out_step = a.tokens;
            } else {
                const int c0 = col * KVC_WAVE;                         // first flat channel of the tile
                const int bh0 = c0 / D;
                const int bh_lane = (c0 + lane) / D;
                const int d = c0 + lane - bh_lane * D;
                const int sel = bh_lane - bh0;                         // 0, or 1 past a head boundary
                float bias_s[2][REP];
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    if (s < slots) {
                        int bh = bh0 + s;
                        const int bh_max = a.batch * a.kv_heads - 1;
                        bh = bh < bh_max ? bh : bh_max;                // slot 1 is unused by a tile that ends the row
                        const int b = bh / a.kv_heads, h = bh - b * a.kv_heads;
#pragma unroll
                        for (int r = 0; r < REP; r++) bias_s[s][r] = 0.f;
#pragma unroll
                        for (int half = 0; half < 2; half++) {
                            const int i = lane + 64 * half;
                            const int64_t tk = (int64_t)row * KVC_V_TOKENS + i;
                            int64_t g;
                            if (a.quant_mask == KVC_MASK_V_TOKEN) g = tk;
                            else if (a.quant_mask == KVC_MASK_SIM_TOKEN) g = tk * a.batch + b;
                            else g = (tk * a.batch + b) * a.kv_heads + h;           // KVC_MASK_VECTOR
                            const float sc = __half2float(a.scale[g]), mn = (float)a.min_i8[g];
#pragma unroll
                            for (int r = 0; r < REP; r++) {
                                const __half *pp = a.x + ((int64_t)b * a.q_heads + h * REP + r) * a.tokens;
                                const float v = sc * __half2float(pp[tk]);
                                ops[(s * 128 + i) * REP + r] = v;
                                bias_s[s][r] += mn * v;
                            }
                        }
#pragma unroll
                        for (int r = 0; r < REP; r++) bias_s[s][r] = kvc_wave_sum(bias_s[s][r]);
                    }
                }
#pragma unroll
                for (int r = 0; r < REP; r++) bias[r] = (slots == 2 && sel) ? bias_s[1][r] : bias_s[0][r];
                my_ops = ops + sel * 128 * REP;
                const int b = bh_lane / a.kv_heads, h = bh_lane - b * a.kv_heads;
                out_base = (((int64_t)row * a.batch + b) * a.q_heads + h * REP) * D + d;
                out_step = D;
            }
            if (IS_K) {
#pragma unroll
                for (int r = 0; r < REP; r++) bias[r] = kvc_wave_sum(bias[r]);
            }
        }
        __syncthreads();
        if (active) {
            float acc[REP];
#pragma unroll
            for (int r = 0; r < REP; r++) acc[r] = 0.f;
            bool redo = !(fast_book && tl.fits);
            if (!redo) {
                uint32_t t = tl.pos + 32u * KVC_STAGE_LEAD_WORDS - 1u, worst = 0;
                const char *fe = reinterpret_cast<const char *>(s_fentry);
                if (lmax <= 4) {
                    kvc_fast_dot<8, false, REP>(stage, last_word, t, fe, mask4, rot, n, my_ops, acc, worst);
                } else if (lmax <= 8) {
                    kvc_fast_dot<4, false, REP>(stage, last_word, t, fe, mask4, rot, n, my_ops, acc, worst);
                } else {
                    kvc_fast_dot<4, true, REP>(stage, last_word, t, fe, mask4, rot, n, my_ops, acc, worst);
                    redo = __any(worst > 32u);
                }
            }
            if (redo) {
                const KvcVec<REP> res = tl.fits
                    ? kvc_slow_tile<REP, false>(stage, (uint32_t)a.stage_words, tl.pos + 32u * KVC_STAGE_LEAD_WORDS, lut_g, n, my_ops)
                    : kvc_slow_tile<REP, true>(tl.gwords, tl.nwords, tl.pos, lut_g, n, my_ops);
#pragma unroll
                for (int r = 0; r < REP; r++) acc[r] = res.v[r];
            }
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const int64_t o = out_base + r * out_step;
                const float v = acc[r] + bias[r];
                if (a.out_f32) reinterpret_cast<float *>(a.out)[o] = v;
                else reinterpret_cast<__half *>(a.out)[o] = __float2half(v);
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------
template <int REP>
static void kvc_launch_fused(int is_k, const KvcFusedArgs &a, dim3 grid, size_t lds, hipStream_t stream)
{
    if (is_k) hipLaunchKernelGGL((kvc_fused_kernel<REP, true>), grid, dim3(KVC_WG), lds, stream, a);
    else hipLaunchKernelGGL((kvc_fused_kernel<REP, false>), grid, dim3(KVC_WG), lds, stream, a);
}

// LDS words per wave for the staged payload: room for about twice the average tile (tiles that still do
// not fit are decoded from global memory), between 1 KiB and the largest tile the format allows.
static int kvc_pick_stage_words(int64_t encoded_bytes, int64_t tiles, int64_t max_tile_bytes)
{
    static int forced = -1;
    if (forced < 0) {
        const char *e = std::getenv("KVC_STAGE_BYTES");
        forced = e ? std::atoi(e) : 0;
    }
    // payload + up to 15 bytes before it in its first chunk, rounded up to chunks, + lead and look-ahead words
    int64_t bytes = max_tile_bytes > 0 ? ((max_tile_bytes + 15 + 15) / 16) * 16 + 4 * (KVC_STAGE_LEAD_WORDS + 2)
                                       : 2 * (encoded_bytes / (tiles > 0 ? tiles : 1)) + 64;
    if (forced > 0) bytes = forced;
    const int64_t max_bytes = ((KVC_MAX_TILE_BYTES + 15 + 15) / 16) * 16 + 16 * KVC_STAGE_LEAD_WORDS / 4 + 16;
    if (bytes < 1024) bytes = 1024;
    if (bytes > max_bytes) bytes = max_bytes;
    bytes = (bytes + 255) / 256 * 256;
    return (int)(bytes / 4);
}

static int kvc_fused(int is_k, const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                     const uint8_t *d_block_infos, int64_t block_infos_bytes, const uint8_t *d_thread_infos,
                     int64_t thread_infos_bytes, const uint8_t *d_encoded, int64_t encoded_bytes,
                     const int8_t *d_min, const void *d_scale, int quant_mask, const void *d_x, void *d_out,
                     int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                     float *elapsed_ms, void *stream_, const uint32_t *d_luts = nullptr, int rows_per_codebook = 0,
                     int out_f32 = 0, int64_t max_tile_bytes = 0)
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
    void *slot = nullptr;
    if (!d_luts) {
        if (int rc = kvc_workspace_slot(&slot)) return rc;
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
    a.tokens = tokens;
    a.batch = (int)batch;
    a.kv_heads = (int)kv_heads;
    a.q_heads = (int)q_heads;
    a.head_dim = (int)head_dim;
    a.stage_words = kvc_pick_stage_words(encoded_bytes, rows * a.s.cols, max_tile_bytes);
    const int slots = (!is_k && head_dim % KVC_WAVE != 0) ? 2 : 1;
    const size_t lds = (size_t)KVC_WAVES_PER_WG * (size_t)(slots * 128 * rep + a.stage_words) * 4;   // operand tables + staging
    KvcTimer timer(elapsed_ms, stream);
    if (!d_luts) {
        if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    }
    const dim3 grid = kvc_grid(a.s, rows);
    switch (rep) {
        case 1: kvc_launch_fused<1>(is_k, a, grid, lds, stream); break;
        case 2: kvc_launch_fused<2>(is_k, a, grid, lds, stream); break;
        case 4: kvc_launch_fused<4>(is_k, a, grid, lds, stream); break;
        default: kvc_launch_fused<8>(is_k, a, grid, lds, stream); break;
    }
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
                                int out_f32, int64_t max_tile_bytes, int64_t tokens, int64_t batch, int64_t kv_heads,
                                int64_t q_heads, int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(1, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_q_f16, d_scores, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32, max_tile_bytes);
}

extern "C" int kvc_v_partials_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                                  int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                  const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                                  const void *d_quant_scales_f16, int quant_mask, const void *d_p_f16, void *d_partial,
                                  int out_f32, int64_t max_tile_bytes, int64_t tokens, int64_t batch, int64_t kv_heads,
                                  int64_t q_heads, int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(0, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_p_f16, d_partial, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32, max_tile_bytes);
}
