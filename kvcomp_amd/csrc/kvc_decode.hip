// kvc_decode.hip -- Huffman tile decoders: plain (symbols back to HBM) and fused with the decode-attention
// matvecs (symbols never leave registers).
//
//   kvc_decode_k_kernel / kvc_decode_v_kernel      <- huffman_decode / v_huffman_decode
//                                                     (kvcomp_cuda_extension/src/kernels.cu:602-719)
//   kvc_fused_k_kernel                             <- huffman_decode_and_mat_vec_mul   (kernels.cu:721-776)
//   kvc_fused_v_kernel                             <- v_huffman_decode_and_mat_vec_mul (kernels.cu:778-861)
//
// Launch shape: grid (ceil(cols / (4 * tiles_per_wave)), tile_rows), 256 threads = 4 waves; each wave
// decodes whole tiles on its own, the workgroup only shares the decode table.  A tile row is the set of
// tiles that cover the same tokens (64 for K, 128 for V), so everything that depends on the token block
// (codebook, block-quant scale) is uniform per workgroup.
#include "kvc_tile.h"

#include <cstdlib>

// ---------------------------------------------------------------------------------------------------
// plain decode
// ---------------------------------------------------------------------------------------------------
constexpr int KVC_KOUT_ROW_WORDS = KVC_K_VEC_LEN / 4 + 1;   // 33: odd stride -> conflict-free column writes

__global__ void __launch_bounds__(KVC_WG) kvc_decode_k_kernel(KvcStreamArgs a, uint8_t *__restrict__ out)
{
    __shared__ uint32_t s_lut[KVC_LUT_WORDS];
    __shared__ __align__(16) uint32_t s_stage[KVC_WAVES_PER_WG][KVC_STAGE_WORDS];
    __shared__ uint32_t s_out[KVC_WAVES_PER_WG][KVC_WAVE * KVC_KOUT_ROW_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.y;
    const int64_t cb = a.rows_per_codebook ? row / a.rows_per_codebook : 0;
    kvc_load_lut(a.luts + cb * KVC_LUT_WORDS, s_lut, tid);
    __syncthreads();
    uint32_t *stage = s_stage[wave];
    uint32_t *tile_out = s_out[wave];
    const int D = a.vec_len;
    for (int it = 0; it < a.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.tiles_per_wave + it;
        const bool active = col < a.cols;
        const int64_t tile = (int64_t)row * a.cols + col;
        uint32_t pos = 0;
        if (active) pos = kvc_stage_tile(a, tile, stage, lane);
        __syncthreads();
        if (active) {
            uint32_t cur = 0;
            auto emit = [&](int i, uint32_t sym) {
                cur |= sym << (8 * (i & 3));
                if ((i & 3) == 3) {
                    tile_out[lane * KVC_KOUT_ROW_WORDS + (i >> 2)] = cur;
                    cur = 0;
                }
            };
            kvc_dispatch_group(s_lut, [&]<int G, bool S>() { kvc_decode_run<G, S>(stage, pos, s_lut, D, emit); });
        }
        __syncthreads();
        if (active) {
            const int dpr = D >> 2;
            uint8_t *base = out + (int64_t)row * KVC_WAVE * a.stride + (int64_t)col * D;
            for (int f = lane; f < KVC_WAVE * dpr; f += KVC_WAVE) {
                const int r = f / dpr, j = f - r * dpr;
                *reinterpret_cast<uint32_t *>(base + (int64_t)r * a.stride + 4 * j) = tile_out[r * KVC_KOUT_ROW_WORDS + j];
            }
        }
        __syncthreads();
    }
}

__global__ void __launch_bounds__(KVC_WG) kvc_decode_v_kernel(KvcStreamArgs a, uint8_t *__restrict__ out)
{
    __shared__ uint32_t s_lut[KVC_LUT_WORDS];
    __shared__ __align__(16) uint32_t s_stage[KVC_WAVES_PER_WG][KVC_STAGE_WORDS];
    __shared__ __align__(16) uint8_t s_out[KVC_WAVES_PER_WG][KVC_V_TOKENS * KVC_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.y;
    const int64_t cb = a.rows_per_codebook ? row / a.rows_per_codebook : 0;
    kvc_load_lut(a.luts + cb * KVC_LUT_WORDS, s_lut, tid);
    __syncthreads();
    uint32_t *stage = s_stage[wave];
    uint8_t *tile_out = s_out[wave];
    for (int it = 0; it < a.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.tiles_per_wave + it;
        const bool active = col < a.cols;
        const int64_t tile = (int64_t)row * a.cols + col;
        uint32_t pos = 0;
        if (active) pos = kvc_stage_tile(a, tile, stage, lane);
        __syncthreads();
        if (active) {
            auto emit = [&](int i, uint32_t sym) { tile_out[i * KVC_WAVE + lane] = (uint8_t)sym; };
            kvc_dispatch_group(s_lut, [&]<int G, bool S>() { kvc_decode_run<G, S>(stage, pos, s_lut, KVC_V_TOKENS, emit); });
        }
        __syncthreads();
        if (active) {
            uint8_t *base = out + (int64_t)row * KVC_V_TOKENS * a.stride + (int64_t)col * KVC_WAVE;
            const uint32_t *w = reinterpret_cast<const uint32_t *>(tile_out);
            for (int f = lane; f < KVC_V_TOKENS * (KVC_WAVE / 4); f += KVC_WAVE) {
                const int i = f >> 4, j = f & 15;
                *reinterpret_cast<uint32_t *>(base + (int64_t)i * a.stride + 4 * j) = w[f];
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------------------------------
// fused decode + matvec
// ---------------------------------------------------------------------------------------------------
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
};

// K: lane <-> token, symbol index <-> channel.
//   score = sum_i (sym_i + min_i) * scale_i * q_i = sum_i sym_i * q'_i + sum_i min_i * q'_i,  q'_i = scale_i * q_i
// q' lives in two VGPRs per query head (lane l holds channels l and l + 64) and reaches the FMA through
// v_readlane, because channel i is the same for every lane.
template <int REP>
__global__ void __launch_bounds__(KVC_WG) kvc_fused_k_kernel(KvcFusedArgs a)
{
    __shared__ uint32_t s_lut[KVC_LUT_WORDS];
    __shared__ __align__(16) uint32_t s_stage[KVC_WAVES_PER_WG][KVC_STAGE_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.y;
    const int64_t cb = a.s.rows_per_codebook ? row / a.s.rows_per_codebook : 0;
    kvc_load_lut(a.s.luts + cb * KVC_LUT_WORDS, s_lut, tid);
    __syncthreads();
    uint32_t *stage = s_stage[wave];
    const int D = a.head_dim;
    const int n0 = D < 64 ? D : 64, n1 = D - n0;
    for (int it = 0; it < a.s.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.s.tiles_per_wave + it;
        const bool active = col < a.s.cols;
        const int64_t tile = (int64_t)row * a.s.cols + col;
        uint32_t pos = 0;
        if (active) pos = kvc_stage_tile(a.s, tile, stage, lane);
        __syncthreads();
        if (active) {
            const int b = col / a.kv_heads, h = col - b * a.kv_heads;
            const int i0 = lane, i1 = lane + 64;
            float sc0, sc1, mn0, mn1;
            if (a.quant_mask == KVC_MASK_CHANNEL) {
                const int64_t g = tile * D;
                sc0 = i0 < D ? __half2float(a.scale[g + i0]) : 0.f;
                sc1 = i1 < D ? __half2float(a.scale[g + i1]) : 0.f;
                mn0 = i0 < D ? (float)a.min_i8[g + i0] : 0.f;
                mn1 = i1 < D ? (float)a.min_i8[g + i1] : 0.f;
            } else {   // KVC_MASK_K_BLOCK: one pair per 64-token block (kernels.cu:771-772)
                sc0 = sc1 = __half2float(a.scale[row]);
                mn0 = mn1 = (float)a.min_i8[row];
            }
            float qa[REP], qb[REP], bias[REP], acc[REP];
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const __half *qp = a.x + ((int64_t)b * a.q_heads + h * REP + r) * D;
                qa[r] = i0 < D ? sc0 * __half2float(qp[i0]) : 0.f;
                qb[r] = i1 < D ? sc1 * __half2float(qp[i1]) : 0.f;
                bias[r] = kvc_wave_sum(mn0 * qa[r] + mn1 * qb[r]);
                acc[r] = 0.f;
            }
            kvc_dispatch_group(s_lut, [&]<int G, bool S>() {
                kvc_decode_run<G, S>(stage, pos, s_lut, n0, [&](int i, uint32_t sym) {
                    const float f = (float)sym;
#pragma unroll
                    for (int r = 0; r < REP; r++) acc[r] = fmaf(f, kvc_readlane(qa[r], i), acc[r]);
                });
                kvc_decode_run<G, S>(stage, pos, s_lut, n1, [&](int i, uint32_t sym) {
                    const float f = (float)sym;
#pragma unroll
                    for (int r = 0; r < REP; r++) acc[r] = fmaf(f, kvc_readlane(qb[r], i), acc[r]);
                });
            });
            const int64_t token = (int64_t)row * KVC_WAVE + lane;
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const int64_t o = ((int64_t)b * a.q_heads + h * REP + r) * a.tokens + token;
                const float v = acc[r] + bias[r];
                if (a.out_f32) reinterpret_cast<float *>(a.out)[o] = v;
                else reinterpret_cast<__half *>(a.out)[o] = __float2half(v);
            }
        }
        __syncthreads();
    }
}

// V: lane <-> channel, symbol index <-> token of the 128-token group.
//   partial = sum_t (sym_t + min_t) * scale_t * p_t = sum_t sym_t * w_t + sum_t min_t * w_t,  w_t = scale_t * p_t
// All 64 channels of a tile belong to one head (head_dim is a multiple of 64), so w_t is uniform.
template <int REP>
__global__ void __launch_bounds__(KVC_WG) kvc_fused_v_kernel(KvcFusedArgs a)
{
    __shared__ uint32_t s_lut[KVC_LUT_WORDS];
    __shared__ __align__(16) uint32_t s_stage[KVC_WAVES_PER_WG][KVC_STAGE_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.y;
    const int64_t cb = a.s.rows_per_codebook ? row / a.s.rows_per_codebook : 0;
    kvc_load_lut(a.s.luts + cb * KVC_LUT_WORDS, s_lut, tid);
    __syncthreads();
    uint32_t *stage = s_stage[wave];
    const int D = a.head_dim;
    for (int it = 0; it < a.s.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.s.tiles_per_wave + it;
        const bool active = col < a.s.cols;
        const int64_t tile = (int64_t)row * a.s.cols + col;
        uint32_t pos = 0;
        if (active) pos = kvc_stage_tile(a.s, tile, stage, lane);
        __syncthreads();
        if (active) {
            const int c0 = col * KVC_WAVE;            // first flat channel of the tile
            const int bh = c0 / D, d = c0 - bh * D + lane;
            const int b = bh / a.kv_heads, h = bh - b * a.kv_heads;
            const int64_t t0 = (int64_t)row * KVC_V_TOKENS + lane, t1 = t0 + 64;
            int64_t g0, g1;
            if (a.quant_mask == KVC_MASK_V_TOKEN) { g0 = t0; g1 = t1; }
            else if (a.quant_mask == KVC_MASK_SIM_TOKEN) { g0 = t0 * a.batch + b; g1 = t1 * a.batch + b; }
            else { g0 = (t0 * a.batch + b) * a.kv_heads + h; g1 = (t1 * a.batch + b) * a.kv_heads + h; }   // KVC_MASK_VECTOR
            const float sc0 = __half2float(a.scale[g0]), sc1 = __half2float(a.scale[g1]);
            const float mn0 = (float)a.min_i8[g0], mn1 = (float)a.min_i8[g1];
            float wa[REP], wb[REP], bias[REP], acc[REP];
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const __half *pp = a.x + ((int64_t)b * a.q_heads + h * REP + r) * a.tokens;
                wa[r] = sc0 * __half2float(pp[t0]);
                wb[r] = sc1 * __half2float(pp[t1]);
                bias[r] = kvc_wave_sum(mn0 * wa[r] + mn1 * wb[r]);
                acc[r] = 0.f;
            }
            kvc_dispatch_group(s_lut, [&]<int G, bool S>() {
                kvc_decode_run<G, S>(stage, pos, s_lut, 64, [&](int i, uint32_t sym) {
                    const float f = (float)sym;
#pragma unroll
                    for (int r = 0; r < REP; r++) acc[r] = fmaf(f, kvc_readlane(wa[r], i), acc[r]);
                });
                kvc_decode_run<G, S>(stage, pos, s_lut, 64, [&](int i, uint32_t sym) {
                    const float f = (float)sym;
#pragma unroll
                    for (int r = 0; r < REP; r++) acc[r] = fmaf(f, kvc_readlane(wb[r], i), acc[r]);
                });
            });
#pragma unroll
            for (int r = 0; r < REP; r++) {
                const int64_t o = (((int64_t)row * a.batch + b) * a.q_heads + h * REP + r) * D + d;
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
static int kvc_tiles_per_wave(int64_t tiles)
{
    static int forced = -1;
    if (forced < 0) {
        const char *e = std::getenv("KVC_TILES_PER_WAVE");
        forced = e ? std::atoi(e) : 0;
    }
    if (forced > 0) return forced;
    return tiles >= 32768 ? 2 : 1;
}

static int kvc_fill_stream_args(KvcStreamArgs &s, const uint8_t *d_encoded, int64_t encoded_bytes,
                                const uint8_t *d_block_infos, int64_t block_infos_bytes,
                                const uint8_t *d_thread_infos, int64_t thread_infos_bytes, const uint32_t *d_luts,
                                int is_k, int64_t tokens, int64_t stride, int64_t head_dim, int64_t *rows_out)
{
    KVC_REQUIRE(head_dim > 0 && head_dim <= KVC_K_VEC_LEN && head_dim % 8 == 0, "head_dim must be a multiple of 8, <= 128");
    KVC_REQUIRE(stride > 0 && stride % 4 == 0, "stride must be a positive multiple of 4");
    int64_t rows, cols;
    if (is_k) {
        KVC_REQUIRE(tokens % KVC_K_VEC_PER_BLK == 0, "K: token count must be a multiple of 64");
        KVC_REQUIRE(stride % head_dim == 0, "K: stride must be a multiple of head_dim");
        rows = tokens / KVC_K_VEC_PER_BLK;
        cols = stride / head_dim;
    } else {
        KVC_REQUIRE(tokens % KVC_V_VEC_LEN == 0, "V: token count must be a multiple of 128");
        KVC_REQUIRE(stride % KVC_V_VEC_PER_BLK == 0, "V: stride must be a multiple of 64");
        rows = tokens / KVC_V_VEC_LEN;
        cols = stride / KVC_V_VEC_PER_BLK;
    }
    KVC_REQUIRE(rows <= 65535, "too many tile rows (%lld) for one launch", (long long)rows);
    KVC_REQUIRE(block_infos_bytes == rows * cols * 8, "block_infos holds %lld bytes, geometry needs %lld",
                (long long)block_infos_bytes, (long long)(rows * cols * 8));
    KVC_REQUIRE(thread_infos_bytes == rows * cols * KVC_WAVE * 2, "thread_infos holds %lld bytes, geometry needs %lld",
                (long long)thread_infos_bytes, (long long)(rows * cols * KVC_WAVE * 2));
    KVC_REQUIRE(((uintptr_t)d_block_infos & 3) == 0 && ((uintptr_t)d_thread_infos & 1) == 0, "metadata pointers misaligned");
    s.enc = d_encoded;
    s.enc_bytes = encoded_bytes;
    s.block_infos = d_block_infos;
    s.thread_infos = reinterpret_cast<const uint16_t *>(d_thread_infos);
    s.luts = d_luts;
    s.rows_per_codebook = 0;
    s.cols = (int)cols;
    s.tiles_per_wave = kvc_tiles_per_wave(rows * cols);
    s.vec_len = is_k ? (int)head_dim : KVC_V_TOKENS;
    s.stride = stride;
    *rows_out = rows;
    return 0;
}

static dim3 kvc_grid(const KvcStreamArgs &s, int64_t rows)
{
    const int per_wg = KVC_WAVES_PER_WG * s.tiles_per_wave;
    return dim3((unsigned)((s.cols + per_wg - 1) / per_wg), (unsigned)rows);
}

static int kvc_entropy_decode(int is_k, const uint8_t *d_encoded, int64_t encoded_bytes, const uint8_t *d_block_infos,
                              int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                              const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format, uint8_t *d_out,
                              int64_t tokens, int64_t stride, int64_t head_dim, float *elapsed_ms, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    if (tokens == 0) {
        if (elapsed_ms) *elapsed_ms = 0.f;
        return 0;
    }
    KVC_REQUIRE(((uintptr_t)d_out & 3) == 0, "output pointer must be 4-byte aligned");
    void *slot;
    if (int rc = kvc_workspace_slot(&slot)) return rc;
    KvcStreamArgs s;
    int64_t rows;
    if (int rc = kvc_fill_stream_args(s, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                                      thread_infos_bytes, (const uint32_t *)slot, is_k, tokens, stride, head_dim, &rows))
        return rc;
    KvcTimer timer(elapsed_ms, stream);
    if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    if (is_k) hipLaunchKernelGGL(kvc_decode_k_kernel, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out);
    else hipLaunchKernelGGL(kvc_decode_v_kernel, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out);
    KVC_HIP(hipGetLastError());
    return timer.finish();
}

extern "C" int kvc_k_entropy_decode(const uint8_t *d_encoded, int64_t encoded_bytes, const uint8_t *d_block_infos,
                                    int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                    const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                    uint8_t *d_out, int64_t tokens, int64_t stride, int64_t head_num, int64_t head_dim,
                                    float *elapsed_ms, void *stream)
{
    (void)head_num;
    return kvc_entropy_decode(1, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                              thread_infos_bytes, d_decode_tree, decode_tree_bytes, tree_format, d_out, tokens, stride,
                              head_dim, elapsed_ms, stream);
}

extern "C" int kvc_v_entropy_decode(const uint8_t *d_encoded, int64_t encoded_bytes, const uint8_t *d_block_infos,
                                    int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                    const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                    uint8_t *d_out, int64_t tokens, int64_t stride, int64_t head_num, int64_t head_dim,
                                    float *elapsed_ms, void *stream)
{
    (void)head_num;
    return kvc_entropy_decode(0, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                              thread_infos_bytes, d_decode_tree, decode_tree_bytes, tree_format, d_out, tokens, stride,
                              head_dim, elapsed_ms, stream);
}

template <int REP>
static void kvc_launch_fused(int is_k, const KvcFusedArgs &a, dim3 grid, hipStream_t stream)
{
    if (is_k) hipLaunchKernelGGL(kvc_fused_k_kernel<REP>, grid, dim3(KVC_WG), 0, stream, a);
    else hipLaunchKernelGGL(kvc_fused_v_kernel<REP>, grid, dim3(KVC_WG), 0, stream, a);
}

static int kvc_fused(int is_k, const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                     const uint8_t *d_block_infos, int64_t block_infos_bytes, const uint8_t *d_thread_infos,
                     int64_t thread_infos_bytes, const uint8_t *d_encoded, int64_t encoded_bytes,
                     const int8_t *d_min, const void *d_scale, int quant_mask, const void *d_x, void *d_out,
                     int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                     float *elapsed_ms, void *stream_, const uint32_t *d_luts = nullptr, int rows_per_codebook = 0,
                     int out_f32 = 0)
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
        KVC_REQUIRE(head_dim % KVC_WAVE == 0, "fused V needs head_dim to be a multiple of 64");
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
    KvcTimer timer(elapsed_ms, stream);
    if (!d_luts) {
        if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    }
    const dim3 grid = kvc_grid(a.s, rows);
    switch (rep) {
        case 1: kvc_launch_fused<1>(is_k, a, grid, stream); break;
        case 2: kvc_launch_fused<2>(is_k, a, grid, stream); break;
        case 4: kvc_launch_fused<4>(is_k, a, grid, stream); break;
        default: kvc_launch_fused<8>(is_k, a, grid, stream); break;
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
                                int out_f32, int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads,
                                int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(1, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_q_f16, d_scores, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32);
}

extern "C" int kvc_v_partials_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                                  int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                  const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                                  const void *d_quant_scales_f16, int quant_mask, const void *d_p_f16, void *d_partial,
                                  int out_f32, int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads,
                                  int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_luts != nullptr, "d_luts is NULL");
    return kvc_fused(0, nullptr, 0, KVC_TREE_I8, d_block_infos, block_infos_bytes, d_thread_infos, thread_infos_bytes,
                     d_encoded, encoded_bytes, d_quant_min_ints, d_quant_scales_f16, quant_mask, d_p_f16, d_partial, tokens,
                     batch, kv_heads, q_heads, head_dim, elapsed_ms, stream, (const uint32_t *)d_luts,
                     (int)rows_per_codebook, out_f32);
}
