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

// What turns the decoded symbols of a tile into fp16 on their way out (DEQ kernels): (sym + min_i) * scale,
// RN16(f32(int) * f32(scale)), models/cache/kvcomp_encode.py:146,161.  Group g of element (token, b, h, d)
// follows the 4-bit mask over (BS, B, H, D) that the quantizer used.
struct KvcDequantArgs {
    const int8_t *min_i8;
    const __half *scale;
    int mask, BS, B, H, D;
};

__device__ __forceinline__ int64_t kvc_group_index(const KvcDequantArgs &q, int64_t token, int b, int h, int d)
{
    const int64_t nb = token / q.BS, bs = token - nb * q.BS;
    const int64_t gBS = (q.mask & 1) ? 1 : q.BS, gB = (q.mask & 2) ? 1 : q.B, gH = (q.mask & 4) ? 1 : q.H, gD = (q.mask & 8) ? 1 : q.D;
    return (((nb * gBS + ((q.mask & 1) ? 0 : bs)) * gB + ((q.mask & 2) ? 0 : b)) * gH + ((q.mask & 4) ? 0 : h)) * gD +
           ((q.mask & 8) ? 0 : d);
}

// four symbols of one token, channels d .. d + 3 of head (b, h) -> four fp16 values
__device__ __forceinline__ uint2 kvc_dequant_word(const KvcDequantArgs &q, uint32_t w, int64_t token, int b, int h, int d)
{
    const int64_t g0 = kvc_group_index(q, token, b, h, d);
    const int64_t step = (q.mask & 8) ? 0 : 1;
    __half o[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t g = g0 + k * step;
        const int v = (int)((w >> (8 * k)) & 0xffu) + (int)q.min_i8[g];
        o[k] = __float2half_rn((float)v * __half2float(q.scale[g]));
    }
    uint2 r;
    r.x = (uint32_t)__half_as_ushort(o[0]) | ((uint32_t)__half_as_ushort(o[1]) << 16);
    r.y = (uint32_t)__half_as_ushort(o[2]) | ((uint32_t)__half_as_ushort(o[3]) << 16);
    return r;
}

// LDS traffic between the lanes of one wave needs no workgroup barrier (a wave's LDS operations complete in
// order); this keeps the compiler from moving accesses across the hand-over.
__device__ __forceinline__ void kvc_decode_wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <bool DEQ>
__global__ void __launch_bounds__(KVC_WG) kvc_decode_k_kernel(KvcStreamArgs a, void *__restrict__ out_, KvcDequantArgs q)
{
    __shared__ uint32_t s_lut[KVC_LUT_WORDS];
    __shared__ __align__(16) uint32_t s_stage[KVC_WAVES_PER_WG][KVC_STAGE_WORDS];
    __shared__ uint32_t s_out[KVC_WAVES_PER_WG][KVC_WAVE * KVC_KOUT_ROW_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.y;
    const int64_t cb = a.rows_per_codebook ? row / a.rows_per_codebook : 0;
    kvc_load_lut(a.luts + cb * KVC_LUT_WORDS, s_lut, tid);
    __syncthreads();
    // from here on every wave works on its own tiles and its own LDS areas
    uint32_t *stage = s_stage[wave];
    uint32_t *tile_out = s_out[wave];
    const int D = a.vec_len;
    for (int it = 0; it < a.tiles_per_wave; it++) {
        const int col = (blockIdx.x * KVC_WAVES_PER_WG + wave) * a.tiles_per_wave + it;
        if (col >= a.cols) break;
        const int64_t tile = (int64_t)row * a.cols + col;
        uint32_t pos = kvc_stage_tile(a, tile, stage, lane);
        kvc_decode_wave_sync();
        uint32_t cur = 0;
        auto emit = [&](int i, uint32_t sym) {
            cur |= sym << (8 * (i & 3));
            if ((i & 3) == 3) {
                tile_out[lane * KVC_KOUT_ROW_WORDS + (i >> 2)] = cur;
                cur = 0;
            }
        };
        kvc_dispatch_group(s_lut, [&]<int G, bool S>() { kvc_decode_run<G, S>(stage, pos, s_lut, D, emit); });
        kvc_decode_wave_sync();
        const int dpr = D >> 2;
        if (DEQ) {
            __half *base = reinterpret_cast<__half *>(out_) + (int64_t)row * KVC_WAVE * a.stride + (int64_t)col * D;
            const int bh = col, b = bh / q.H, h = bh - b * q.H;
            for (int f = lane; f < KVC_WAVE * dpr; f += KVC_WAVE) {
                const int r = f / dpr, j = f - r * dpr;
                const uint2 v = kvc_dequant_word(q, tile_out[r * KVC_KOUT_ROW_WORDS + j], (int64_t)row * KVC_WAVE + r, b, h, 4 * j);
                *reinterpret_cast<uint2 *>(base + (int64_t)r * a.stride + 4 * j) = v;
            }
        } else {
            uint8_t *base = reinterpret_cast<uint8_t *>(out_) + (int64_t)row * KVC_WAVE * a.stride + (int64_t)col * D;
            for (int f = lane; f < KVC_WAVE * dpr; f += KVC_WAVE) {
                const int r = f / dpr, j = f - r * dpr;
                *reinterpret_cast<uint32_t *>(base + (int64_t)r * a.stride + 4 * j) = tile_out[r * KVC_KOUT_ROW_WORDS + j];
            }
        }
        kvc_decode_wave_sync();
    }
}

template <bool DEQ>
__global__ void __launch_bounds__(KVC_WG) kvc_decode_v_kernel(KvcStreamArgs a, void *__restrict__ out_, KvcDequantArgs q)
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
        if (col >= a.cols) break;
        const int64_t tile = (int64_t)row * a.cols + col;
        uint32_t pos = kvc_stage_tile(a, tile, stage, lane);
        kvc_decode_wave_sync();
        auto emit = [&](int i, uint32_t sym) { tile_out[i * KVC_WAVE + lane] = (uint8_t)sym; };
        kvc_dispatch_group(s_lut, [&]<int G, bool S>() { kvc_decode_run<G, S>(stage, pos, s_lut, KVC_V_TOKENS, emit); });
        kvc_decode_wave_sync();
        const uint32_t *w = reinterpret_cast<const uint32_t *>(tile_out);
        if (DEQ) {
            __half *base = reinterpret_cast<__half *>(out_) + (int64_t)row * KVC_V_TOKENS * a.stride + (int64_t)col * KVC_WAVE;
            // lane l always handles channels 4 (l & 15) .. + 3 of the tile: its head and channel are fixed
            const int c = col * KVC_WAVE + 4 * (lane & 15);
            const int bh = c / q.D, d = c - bh * q.D, b = bh / q.H, h = bh - b * q.H;
            for (int f = lane; f < KVC_V_TOKENS * (KVC_WAVE / 4); f += KVC_WAVE) {
                const int i = f >> 4, j = f & 15;
                const uint2 v = kvc_dequant_word(q, w[f], (int64_t)row * KVC_V_TOKENS + i, b, h, d);
                *reinterpret_cast<uint2 *>(base + (int64_t)i * a.stride + 4 * j) = v;
            }
        } else {
            uint8_t *base = reinterpret_cast<uint8_t *>(out_) + (int64_t)row * KVC_V_TOKENS * a.stride + (int64_t)col * KVC_WAVE;
            for (int f = lane; f < KVC_V_TOKENS * (KVC_WAVE / 4); f += KVC_WAVE) {
                const int i = f >> 4, j = f & 15;
                *reinterpret_cast<uint32_t *>(base + (int64_t)i * a.stride + 4 * j) = w[f];
            }
        }
        kvc_decode_wave_sync();
    }
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------
static int kvc_entropy_decode(int is_k, const uint8_t *d_encoded, int64_t encoded_bytes, const uint8_t *d_block_infos,
                              int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                              const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format, void *d_out,
                              int64_t tokens, int64_t stride, int64_t head_dim, float *elapsed_ms, void *stream_,
                              const KvcDequantArgs *deq = nullptr)
{
    hipStream_t stream = (hipStream_t)stream_;
    if (tokens == 0) {
        if (elapsed_ms) *elapsed_ms = 0.f;
        return 0;
    }
    KVC_REQUIRE(((uintptr_t)d_out & (deq ? 7 : 3)) == 0, "output pointer is misaligned");
    // the pipelined kernel (kvc_fused.hip) handles the usual layouts; 1 = not this one
    if (kvc_option(KVC_OPT_DECODE_PIPELINED) && ((uintptr_t)d_out & 15) == 0 && stride % head_dim == 0 &&
        (!deq || !is_k || deq->BS == KVC_K_VEC_PER_BLK)) {
        const int64_t heads_x_batch = stride / head_dim;
        const int rc = deq ? kvc_expand(is_k, 1, d_decode_tree, decode_tree_bytes, tree_format, d_block_infos, block_infos_bytes,
                                        d_thread_infos, thread_infos_bytes, d_encoded, encoded_bytes, deq->min_i8, deq->scale,
                                        deq->mask, d_out, tokens, deq->B, deq->H, head_dim, elapsed_ms, stream_)
                           : kvc_expand(is_k, 0, d_decode_tree, decode_tree_bytes, tree_format, d_block_infos, block_infos_bytes,
                                        d_thread_infos, thread_infos_bytes, d_encoded, encoded_bytes, nullptr, nullptr, 0, d_out,
                                        tokens, 1, heads_x_batch, head_dim, elapsed_ms, stream_);
        if (rc != 1) return rc;
    }
    void *slot;
    if (int rc = kvc_workspace_slot(&slot, (void *)stream_)) return rc;
    KvcStreamArgs s;
    int64_t rows;
    if (int rc = kvc_fill_stream_args(s, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                                      thread_infos_bytes, (const uint32_t *)slot, is_k, tokens, stride, head_dim, &rows))
        return rc;
    KvcTimer timer(elapsed_ms, stream);
    if (int rc = kvc_launch_build_lut(d_decode_tree, decode_tree_bytes, tree_format, (uint32_t *)slot, 1, 0, stream)) return rc;
    const KvcDequantArgs q = deq ? *deq : KvcDequantArgs{nullptr, nullptr, 0, 1, 1, 1, 1};
    if (is_k && deq) hipLaunchKernelGGL(kvc_decode_k_kernel<true>, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out, q);
    else if (is_k) hipLaunchKernelGGL(kvc_decode_k_kernel<false>, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out, q);
    else if (deq) hipLaunchKernelGGL(kvc_decode_v_kernel<true>, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out, q);
    else hipLaunchKernelGGL(kvc_decode_v_kernel<false>, kvc_grid(s, rows), dim3(KVC_WG), 0, stream, s, d_out, q);
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


// ---------------------------------------------------------------------------------------------------
// decode + dequantize in one pass: KVCompCtx.get_only_compressed (models/cache/kvcomp_encode.py:153-166)
// without the uint8 symbol tensor in between
// ---------------------------------------------------------------------------------------------------
extern "C" int kvc_decode_dequant(int is_k, const uint8_t *d_encoded, int64_t encoded_bytes, const uint8_t *d_block_infos,
                                  int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                  const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                  const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                                  int64_t block_size, void *d_out_f16, int64_t tokens, int64_t batch, int64_t heads,
                                  int64_t head_dim, float *elapsed_ms, void *stream)
{
    KVC_REQUIRE(d_quant_min_ints != nullptr && d_quant_scales_f16 != nullptr && d_out_f16 != nullptr, "NULL argument");
    KVC_REQUIRE((quant_mask & ~0xF) == 0, "bad quantization group mask");
    KVC_REQUIRE(block_size > 0 && tokens % block_size == 0, "token count must be whole quantization blocks");
    KVC_REQUIRE(batch > 0 && heads > 0 && head_dim > 0 && head_dim % 4 == 0, "bad shape");
    const KvcDequantArgs q = {d_quant_min_ints, reinterpret_cast<const __half *>(d_quant_scales_f16), quant_mask,
                              (int)block_size, (int)batch, (int)heads, (int)head_dim};
    return kvc_entropy_decode(is_k, d_encoded, encoded_bytes, d_block_infos, block_infos_bytes, d_thread_infos,
                              thread_infos_bytes, d_decode_tree, decode_tree_bytes, tree_format, d_out_f16, tokens,
                              batch * heads * head_dim, head_dim, elapsed_ms, stream, &q);
}
