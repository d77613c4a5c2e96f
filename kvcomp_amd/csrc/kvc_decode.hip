// kvc_decode.hip -- Huffman tile decoders: plain (symbols back to HBM) and fused with the decode-attention
// matvecs.
//
//   kvc_decode_k_kernel / kvc_decode_v_kernel      <- huffman_decode / v_huffman_decode
//                                                     (kvcomp_cuda_extension/src/kernels.cu:602-719)
// (the fused decode + matvec kernels live in kvc_fused.hip)
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
// host side
// ---------------------------------------------------------------------------------------------------
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

