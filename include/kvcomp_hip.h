/*
 * kvcomp_hip.h -- C ABI of libkvcomp_hip.so: KVComp's KV-cache codec and compressed decode-attention
 * path for AMD MI355X (gfx950), written directly in HIP.
 *
 * The entry points below are what a binding of the reference's `kvcomp_cuda` operator module
 * (kvcomp_cuda_extension/export_kvcomp.cpp:8-26, signatures in kvcomp_cuda_extension/kvcomp_cuda.pyi)
 * needs: plain device/host pointers and sizes, no framework types.  Each declaration cites the
 * reference interface it replaces (paths relative to the reference checkout).
 *
 * Conventions
 *   - d_* pointers are device memory on the CURRENT HIP device, h_* pointers are host memory.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls are asynchronous
 *     on that stream unless stated otherwise.
 *   - Return value 0 = success; negative = error, with a message from kvc_last_error() (thread local).
 *     The reference aborts the process on a failed check (include/utils.h:7-15); this library returns
 *     an error instead so a host language can raise.
 *   - Symbol tensors are uint8 [NB, BS, B, H, D] contiguous: `tokens` = NB*BS, `stride` = B*H*D bytes
 *     per token (kvcomp_cuda_extension/src/kernels.cu:939,986).
 *   - Tile geometry (kernels.cu:431-444, 503-519, include/kernels.h:12-19):
 *       K tile = 64 tokens x head_dim channels of one (b,h); lane t <-> token      (head_dim <= 128;
 *                the reference requires head_dim == 128)
 *       V tile = 128 tokens x 64 adjacent flat channels;     lane t <-> channel
 *   - Wire structs (include/kernels.h:25-42, include/huffman.h:13-22), little-endian:
 *       block_info  {u32 offset; u16 byte_num; u16 pad}  8 B per tile
 *       thread_info {u16 end_byte*8 + pad_bits}          2 B per lane stream
 *       encode table entry {u32 code; u32 length}        8 B per symbol, index = symbol
 *       decode tree node   {u8 is_leaf; i8 a; i8 b}      3 B
 *     Tile payloads are laid out in tile order (the reference claims offsets with a global atomic in
 *     arrival order, kernels.cu:472-479); every per-tile quantity is identical to the reference's.
 */
#ifndef KVCOMP_HIP_H
#define KVCOMP_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* export_kvcomp.cpp:9-12 / include/kernels.h:12-19 */
#define KVC_K_VEC_LEN 128
#define KVC_K_VEC_PER_BLK 64
#define KVC_V_VEC_LEN 128
#define KVC_V_VEC_PER_BLK 64

/* (min, scale) group descriptor of the quantizer: bit set = that dimension of [NB, BS, B, H, D] is
 * reduced over (BS = 1, B = 2, H = 4, D = 8).  NB is never reduced. */
#define KVC_MASK_K_BLOCK 0xF   /* models/cache/kvcomp_encode.py:10-13  BlockQuant dims [1,2,3,4] */
#define KVC_MASK_V_TOKEN 0xE   /* models/cache/kvcomp_encode.py:10-13  TokenQuant dims [2,3,4]   */
#define KVC_MASK_CHANNEL 0x1   /* utils/compute.py:140  ChannelQuant                             */
#define KVC_MASK_SIM_TOKEN 0xC /* utils/compute.py:141  TokenQuant on [B,H,NB,BS,D]              */
#define KVC_MASK_VECTOR 0x8    /* utils/compute.py:142  VectorQuant                              */
#define KVC_MASK_SIM_BLOCK 0xD /* utils/compute.py:139  BlockQuant on [B,H,NB,BS,D]              */

/* Decode-tree node formats accepted by the decoders. */
#define KVC_TREE_I8 3          /* the reference's 3-byte node (<= 127 nodes, symbols <= 127)      */
#define KVC_TREE_I16 5         /* {u8 is_leaf; i16 a; i16 b}: same walk, lifts both limits        */

const char *kvc_last_error(void);
int kvc_abi_version(void);
/* Tuning knobs (no counterpart in the reference).  Each can also be preset through the environment
 * variable KVCOMP_<NAME IN CAPITALS>, read once on first use.
 *   "fused_rows":           1: the fused decoders re-lay a tile's lane streams as LDS rows an odd number of words
 *                           apart whenever they fit; otherwise (default -1) never.
 *   "fused_skew":           -1 (default) decided per call: the tile payload is staged with two spare words after
 *                           every 32 when the mean stream length would otherwise line the lanes up on a few LDS
 *                           banks; 0 never; 1 always.
 *   "fused_tiles_per_wave":  0 (default) chosen per call; n > 0: consecutive tiles one wave works through.
 *   "fused_pair_bits":       widest index of the two-symbols-per-look-up table (default 8; 0 = one symbol per look-up).
 *   "fused_double_window":   1 (default): 64 stream bits per refill in the one-symbol loops; 0: 32.
 *   "fused_rounded":         1 (default): the fused matvecs round every (sym + min) * scale to fp16 before it meets
 *                           q / p, as the reference's dequantizer rounds it (models/cache/kvcomp_encode.py:146), so the
 *                           result is the fp32 attention over that fp16 cache (within 1e-3).  0: the product is used
 *                           as it stands, in fp32 (closer to exact arithmetic over the unrounded dequantization, and
 *                           further from the reference's cache: a few 1e-3 on outlier-heavy data).
 *   "fused_mfma":           -1 (default) or 1: the multiply-accumulate of the fused matvecs runs on the matrix cores
 *                           (v_mfma_f32_4x4x4_16b_f16) wherever those kernels apply (codes of at most 7 bits, results
 *                           that can be stored four at a time); 0: never (fp32 multiply-adds on the vector units).
 *   "fused_half_table":      1 (default): for codes of 6 or 7 bits the matrix-core kernels use two-byte decode table entries
 *                           (64 entries = one LDS word per bank); 0: four-byte entries.
 *   "fused_builtin_dpp":     0 (default): the fp32-FMA kernels pick their operand out of a quad of lanes with a permute
 *                           written as inline assembly on the multiply-add itself; 1: through the compiler's lane-
 *                           permute intrinsic (same result bit for bit; a cross-check against toolchain changes).
 *   "fused_schedule":       -1 (default) decided per call: a matrix-core launch over a stream with one codebook and at
 *                           least 32768 tiles walks the row-major tile sequence with runs of 4 tiles per wave for the
 *                           first 70 % of the tiles, 2 for the next 20 %, single tiles last; 0: never (every wave
 *                           takes "fused_tiles_per_wave" tiles of one tile row); r * 10000 + p * 100 + q: runs of r
 *                           for the first p %, r / 2 for the next q %, r / 4 and 1 for halves of the rest.
 *   "encode_one_pass":       1 (default): the fused quantize + encode (kvc_store_fused, kvc_encode_async from fp16) reads
 *                           its input once: a wave quantizes and counts its tiles, finds their place in the payload by looking back
 *                           over the sizes the tiles before it have published, and emits them; so do encodes from uint8
 *                           symbols of at least 8192 tiles.  0: two passes (count, offsets, emit), also taken when
 *                           block_infos is not 8-byte aligned or the call has more than 84 224 tiles, and by the other
 *                           encoders that start from uint8 symbols; 2 / 3: one pass for every encoder, with
 *                           always one / two tiles per wave.  Same bytes either way.
 *   "encode_lookback_polls": how often a wave of the one-pass encoder asks again for a size that an earlier tile has not
 *                           published yet before it gives the call up (default 262144; a wave normally asks 50 - 60
 *                           times at most, reported in d_result[6]).  Workgroups take their tiles by a ticket drawn when
 *                           they start, so what a wave waits for has always started before it; a call that is given up
 *                           all the same is encoded again by one workgroup in two passes inside the same launch
 *                           sequence (same bytes, no error, 50 - 100 x slower).  0: every wait gives up at once, -1:
 *                           every call is treated as given up -- both only drive that path from a test.
 *   "fused_schedule_v", "fused_tiles_per_wave_v": -1 (default): as "fused_schedule" / "fused_tiles_per_wave"; other
 *                           values apply to the V kernels only (whose runs follow the head pattern: a run of the
 *                           default schedule is a multiple of lcm(head_dim, 64) / 64 tiles, so that the tiles of a run
 *                           share their heads' operand tables).
 *   "attention_tail_in_merge": 1 (default): kvc_attention_decode handles V's fp16 tail (up to 1024 tokens, K compressed
 *                           at least as far as V) inside its merge kernel; 0: with two kernels of its own.
 *   "decode_pipelined":      1 (default): plain decode and decode + dequantize run on the fused kernels' tile
 *                           pipeline; 0: on the simpler stand-alone kernels. */
int kvc_set_option(const char *name, int value);
int kvc_get_option(const char *name, int *value);

/* ---- sizes: calculate_buffer_size (kernels.cu:893-917) --------------------------------------------
 * out4 = {block_infos bytes, thread_infos bytes, idx_offset bytes (8), payload pre-allocation bytes}. */
int kvc_calculate_buffer_size(int64_t tokens, int64_t stride, int is_k, int64_t head_num, int64_t head_dim,
                              int64_t out4[4]);

/* ---- codebook: build_codebook (src/huffman.cpp:99-157) --------------------------------------------
 * kvc_histogram: 256-bin counts of n device symbols, ADDED into d_counts (int64[256], device).
 * kvc_build_codebook_host: Huffman tree from counts (min-heap on frequency only, ties resolved exactly
 *   as std::priority_queue / heapq do, src/huffman.cpp:34-96) -> shift (= smallest symbol), the encode
 *   table (src/huffman.cpp:166-187) and the decode tree (src/huffman.cpp:229-252) as host bytes.
 *   tree_format KVC_TREE_I8 reproduces the reference bytes and fails if they cannot represent the code
 *   (> 127 nodes, symbol > 127, lone symbol); KVC_TREE_I16 always works for >= 2 symbols. */
int kvc_histogram(const uint8_t *d_sym, int64_t n, int64_t *d_counts, void *stream);
int kvc_build_codebook_host(const int64_t *h_counts256, int tree_format, int *shift,
                            uint8_t *h_encode_table, int64_t encode_cap, int64_t *encode_bytes,
                            uint8_t *h_decode_tree, int64_t decode_cap, int64_t *decode_bytes);

/* The same on the device, for n_codebooks codebooks in one launch and without a host round trip (the reference
 * builds every codebook on the host, src/huffman.cpp:99-157, after 256 .item() reads).
 * kvc_histogram_chunks: one histogram per chunk of chunk_bytes symbols (e.g. the 64-token blocks of a per-block
 *   codebook), ADDED into d_counts (int64[n_chunks][256]).
 * kvc_build_codebook_device: d_counts int64[n][256] ->
 *   d_encode_tables  n x 2048 bytes: the reference's table ({u32 code; u32 length}, entry i = symbol shift + i),
 *                    zero beyond its (largest - smallest symbol + 1) entries;
 *   d_decode_trees   n x kvc_codebook_tree_capacity(tree_format) bytes: the reference's node array, followed by
 *                    childless inner nodes up to the capacity (pass the capacity as tree_bytes to kvc_build_lut);
 *   d_meta           int32[n][4] = {shift, encode table bytes, decode tree bytes, status}; status 0 = built,
 *                    1 = fewer than two distinct symbols, 2 = a code exceeds 32 bits, 4 = not representable in the
 *                    int8 tree (more than 128 nodes or a symbol above 127): then both sizes are 0 and the tables
 *                    hold no code.  Bytes are identical to what kvc_build_codebook_host returns. */
int64_t kvc_codebook_tree_capacity(int tree_format);
int kvc_histogram_chunks(const uint8_t *d_sym, int64_t chunk_bytes, int64_t n_chunks, int64_t *d_counts, void *stream);
int kvc_build_codebook_device(const int64_t *d_counts, int64_t n_codebooks, int tree_format, uint8_t *d_encode_tables,
                              uint8_t *d_decode_trees, int32_t *d_meta, void *stream);

/* ---- encode: k_/v_entropy_encode_cuda_export (kernels.cu:919-1011) --------------------------------
 * Writes block_infos (tiles*8 B), thread_infos (tiles*64*2 B) and the payload; *h_total_bytes receives
 * the payload size (the reference returns encoded_data[:total]).  Synchronises the stream before
 * returning, like the reference's cudaDeviceSynchronize.  d_idx_offset (8 B) receives
 * {u32 tiles, u32 bytes} as in include/kernels.h:34-42.  block_info.offset = base_global_offset +
 * offset inside this call's payload.  Fails if a tile payload exceeds 8191 B (thread_info is u16) or
 * the payload exceeds encoded_cap.  *h_max_tile_bytes / *h_max_stream_bytes (each may be NULL) receive the
 * largest tile payload and the longest single lane stream of this call, which the table-driven fused
 * decoders accept as sizing hints. */
int kvc_k_entropy_encode(const uint8_t *d_sym, int64_t tokens, int64_t stride,
                         const uint8_t *d_encode_table, int64_t encode_table_bytes,
                         uint8_t *d_block_infos, uint8_t *d_thread_infos, uint8_t *d_idx_offset,
                         uint8_t *d_encoded, int64_t encoded_cap, uint32_t base_global_offset,
                         int64_t head_num, int64_t head_dim, int64_t *h_total_bytes,
                         int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream);
int kvc_v_entropy_encode(const uint8_t *d_sym, int64_t tokens, int64_t stride,
                         const uint8_t *d_encode_table, int64_t encode_table_bytes,
                         uint8_t *d_block_infos, uint8_t *d_thread_infos, uint8_t *d_idx_offset,
                         uint8_t *d_encoded, int64_t encoded_cap, uint32_t base_global_offset,
                         int64_t head_num, int64_t head_dim, int64_t *h_total_bytes,
                         int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream);

/* ---- fused quantize + encode ---------------------------------------------------------------------------
 * The store path of models/cache/kvcomp_encode.py:86-112 (quant, the int8 / uint8 casts, k_/v_entropy_encode)
 * as one call straight from the fp16 cache rows: d_x_f16 is [tokens, batch, heads, head_dim] fp16, both encoder
 * passes quantize their tile on the fly, so no symbol tensor is written or read.  Outputs are exactly those of
 * kvc_quant followed by kvc_k_/v_entropy_encode: min_i8 / scale_f16 with the group layout of quant_mask (64-token
 * blocks), thread_infos, block_infos, payload, idx_offset and the three host totals.
 * Layouts: K with KVC_MASK_CHANNEL or KVC_MASK_K_BLOCK; V with KVC_MASK_V_TOKEN, or KVC_MASK_SIM_TOKEN when
 * heads * head_dim is a multiple of 64 (kvc_store_fused_supported says which; others use the two-call path). */
int kvc_store_fused_supported(int is_k, int quant_mask, int64_t batch, int64_t heads, int64_t head_dim);
int kvc_store_fused(int is_k, const void *d_x_f16, int64_t tokens, int64_t batch, int64_t heads, int64_t head_dim,
                    int quant_mask, float eb, const uint8_t *d_encode_table, int64_t encode_table_bytes,
                    int8_t *d_min_i8, void *d_scale_f16, uint8_t *d_block_infos, uint8_t *d_thread_infos,
                    uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap, uint32_t base_global_offset,
                    int64_t *h_total_bytes, int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream);

/* ---- encode without a host round trip (no counterpart in the reference: its encoder copies its counters to the host
 * and waits for the device on every call, kernels.cu:950-965, and takes one codebook per call) -------------------
 * kvc_encode_async queues one encode (from symbols, or -- d_sym == NULL -- quantizing d_x_f16 on the fly exactly as
 * kvc_store_fused does) and returns without waiting; nothing in it is a memset, so it can be recorded in a HIP graph.
 *   codebooks   n tables as kvc_build_codebook_device writes them, table_stride_bytes apart; tile row r (64 tokens of K,
 *               128 of V) is encoded with table r / rows_per_codebook (0: one table for every row).  With
 *               d_codebook_meta (that builder's int32[n][4]) a table that was not built flags the call.
 *   placement   d_stream_bytes == NULL: the payload goes to d_encoded[0 ..) and block_info.offset = base_global_offset +
 *               position, as in kvc_k_/v_entropy_encode.  Otherwise *d_stream_bytes (device, in / out) says how many
 *               payload bytes d_encoded already holds: the call appends behind them, offsets continue from there, and
 *               on success the counter moves on -- so successive calls need no size from the host.
 *   d_result    device uint32[8], zeroed once by the caller, then shared by successive calls:
 *               [0] payload bytes of the latest call, [1] error bits of all calls so far (0 = none), [2] largest tile
 *               payload and [3] longest lane stream so far (sizing hints of the fused decoders), [4] tiles encoded
 *               so far, [5] block_info.offset of the latest call's first tile, [6] the most look-back polls any wave of
 *               any one-pass call so far needed (see "encode_lookback_polls"), [7] reserved.
 * Scratch memory: encodes, the fused matvecs and kvc_attention_decode take 16 KiB slots of a per-device pool, handed out
 * in turn per call (32 slots) -- except under stream capture (hipStreamIsCapturing), where every recorded call gets a
 * slot of its own that is never handed out again (480 such slots per device; beyond them the call fails with a
 * message), so replays of a graph never share scratch memory with later eager calls.  The pool is allocated by the
 * first call on a device, which therefore must not be a recorded one.
 * kvc_encode_result copies d_result to the host (it waits for the stream), turns error bits into an error return
 * and hands out the figures (any pointer may be NULL). */
typedef struct kvc_encode_job {
    int32_t is_k;
    int32_t quant_mask;               /* d_sym == NULL: layout of the (min, scale) groups, as for kvc_store_fused */
    const uint8_t *d_sym;             /* uint8 [tokens, batch * heads * head_dim], or NULL */
    const void *d_x_f16;              /* d_sym == NULL: fp16 [tokens, batch, heads, head_dim] */
    float eb;
    int8_t *d_min_i8;                 /* d_sym == NULL: quantizer outputs */
    void *d_scale_f16;
    int64_t tokens, batch, heads, head_dim;
    const uint8_t *d_encode_tables;
    int64_t encode_table_bytes;       /* bytes of a table that hold entries (at most 2048) */
    int64_t table_stride_bytes;
    int64_t rows_per_codebook;
    const int32_t *d_codebook_meta;   /* may be NULL */
    uint8_t *d_block_infos;
    uint8_t *d_thread_infos;
    uint8_t *d_encoded;
    int64_t encoded_cap;
    uint32_t base_global_offset;
    uint32_t *d_stream_bytes;         /* may be NULL */
    uint32_t *d_result;               /* may be NULL if d_stream_bytes is not */
} kvc_encode_job;
int kvc_encode_async(const kvc_encode_job *job, void *stream);
int kvc_encode_result(const uint32_t *d_result, int64_t encoded_cap, int64_t *h_total_bytes, int64_t *h_max_tile_bytes,
                      int64_t *h_max_stream_bytes, int64_t *h_tiles, void *stream);

/* ---- decode: k_/v_entropy_decode_cuda_export (kernels.cu:1013-1087) -------------------------------
 * d_out uint8 [tokens, stride].  If elapsed_ms != NULL the kernel is bracketed by events, the call
 * waits for it and stores the elapsed milliseconds (the reference's return value); otherwise the call
 * is asynchronous. */
int kvc_k_entropy_decode(const uint8_t *d_encoded, int64_t encoded_bytes,
                         const uint8_t *d_block_infos, int64_t block_infos_bytes,
                         const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                         const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                         uint8_t *d_out, int64_t tokens, int64_t stride,
                         int64_t head_num, int64_t head_dim, float *elapsed_ms, void *stream);
int kvc_v_entropy_decode(const uint8_t *d_encoded, int64_t encoded_bytes,
                         const uint8_t *d_block_infos, int64_t block_infos_bytes,
                         const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                         const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                         uint8_t *d_out, int64_t tokens, int64_t stride,
                         int64_t head_num, int64_t head_dim, float *elapsed_ms, void *stream);

/* ---- decode + dequantize: KVCompCtx.get_only_compressed (models/cache/kvcomp_encode.py:153-166) -----
 * The decoder above followed by (sym + min_i) * scale (kvcomp_encode.py:161) in the same kernel: d_out_f16 is
 * fp16 [tokens, batch, heads, head_dim] = RN16(f32(sym + min_i) * f32(scale)), bit for bit what the two steps
 * give, without the uint8 tensor in between.  quant_mask / block_size say how (min, scale) are grouped
 * (any KVC_MASK_* layout). */
int kvc_decode_dequant(int is_k, const uint8_t *d_encoded, int64_t encoded_bytes,
                       const uint8_t *d_block_infos, int64_t block_infos_bytes,
                       const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                       const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                       const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                       int64_t block_size, void *d_out_f16, int64_t tokens, int64_t batch, int64_t heads,
                       int64_t head_dim, float *elapsed_ms, void *stream);

/* ---- fused decode + matvec: k_/v_decode_and_mat_vec_mul_cuda_export (kernels.cu:1093-1180) --------
 * K: d_q fp16 [batch, q_heads, head_dim]; d_scores fp16 [batch, q_heads, tokens]:
 *      scores[b,hq,t] = sum_i dequant(K[t,b,hq/rep,i]) * q[b,hq,i]          (kernels.cu:721-776)
 * V: d_p fp16 [batch, q_heads, tokens]; d_partial fp16 [tokens/128, batch, q_heads, head_dim]:
 *      partial[g,b,hq,d] = sum_{t<128} dequant(V[128g+t,b,hq/rep,d]) * p[b,hq,128g+t]
 *    (kernels.cu:778-861; the caller sums over g, models/cache/kvcomp_encode.py:275)
 * quant_mask selects the (min, scale) layout: the reference's kernels take KVC_MASK_K_BLOCK for K
 * (kernels.cu:771-772) and KVC_MASK_V_TOKEN for V (kernels.cu:822-833); K also accepts
 * KVC_MASK_CHANNEL (min/scale per (block, b, h, channel)).  q_heads must be a multiple of kv_heads
 * (the reference has q_heads == kv_heads).  Decoded symbols stay in registers; accumulation is fp32
 * (the reference accumulates in fp16, kernels.cu:321,378).  elapsed_ms as for decode. */
int kvc_k_decode_and_mat_vec_mul(const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                 const uint8_t *d_block_infos, int64_t block_infos_bytes,
                                 const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                 const uint8_t *d_encoded, int64_t encoded_bytes,
                                 const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                                 const void *d_q_f16, void *d_scores_f16,
                                 int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                                 float *elapsed_ms, void *stream);
int kvc_v_decode_and_mat_vec_mul(const uint8_t *d_decode_tree, int64_t decode_tree_bytes, int tree_format,
                                 const uint8_t *d_block_infos, int64_t block_infos_bytes,
                                 const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                                 const uint8_t *d_encoded, int64_t encoded_bytes,
                                 const int8_t *d_quant_min_ints, const void *d_quant_scales_f16, int quant_mask,
                                 const void *d_p_f16, void *d_partial_f16,
                                 int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                                 float *elapsed_ms, void *stream);

/* ---- decode tables built once (no counterpart in the reference, which walks its tree bit by bit) ----
 * The decoders look symbols up in a table derived from the decode tree.  The reference-signature entry
 * points above derive it on every call; these take tables prepared once per codebook:
 *   kvc_build_lut: n_codebooks trees, tree_stride_bytes apart, each tree_bytes long -> d_luts
 *                  (n_codebooks * kvc_lut_bytes() bytes, 16-byte aligned).
 *   kvc_k_scores_lut / kvc_v_partials_lut: as kvc_k_/v_decode_and_mat_vec_mul, plus
 *     rows_per_codebook: tile rows (64 tokens for K, 128 for V) that share one table; 0 = one table for all
 *     out_f32:           1 writes fp32 results instead of fp16
 *     max_tile_bytes, max_stream_bytes:
 *                        largest tile payload / longest lane stream in the payload (from the encoder),
 *                        0 = unknown.  They only size the LDS staging; tiles that exceed them are decoded
 *                        from global memory.
 *     max_code_bits:     longest code of the codebook(s), 0 = unknown.  It only sizes the table kept in LDS
 *                        (fewer bytes, more waves per CU); a codebook with longer codes than stated still
 *                        decodes correctly, on the slow path. */
int64_t kvc_lut_bytes(void);
int kvc_build_lut(const uint8_t *d_decode_trees, int64_t tree_bytes, int tree_format, int64_t n_codebooks,
                  int64_t tree_stride_bytes, void *d_luts, void *stream);
int kvc_k_scores_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                     int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                     const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                     const void *d_quant_scales_f16, int quant_mask, const void *d_q_f16, void *d_scores,
                     int out_f32, int64_t max_tile_bytes, int64_t max_stream_bytes, int max_code_bits,
                     int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                     float *elapsed_ms, void *stream);
int kvc_v_partials_lut(const void *d_luts, int64_t rows_per_codebook, const uint8_t *d_block_infos,
                       int64_t block_infos_bytes, const uint8_t *d_thread_infos, int64_t thread_infos_bytes,
                       const uint8_t *d_encoded, int64_t encoded_bytes, const int8_t *d_quant_min_ints,
                       const void *d_quant_scales_f16, int quant_mask, const void *d_p_f16, void *d_partial,
                       int out_f32, int64_t max_tile_bytes, int64_t max_stream_bytes, int max_code_bits,
                       int64_t tokens, int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                       float *elapsed_ms, void *stream);

/* ---- decode attention in one call (no counterpart in the reference: its models decompress the whole cache and
 * run dense attention, models/cache/kvcomp_quant.py:74-75) ----------------------------------------------------
 * out[b, hq, :] = softmax_t(softmax_scale * q[b, hq, :] . K[t, b, h, :]) . V[t, b, h, :] over every stored token:
 * the compressed parts of K and V through the fused kernels, their fp16 tails (the most recent tokens, which K
 * and V keep in different numbers) densely.  A kvc_compressed_desc describes one tensor of the pair: the same
 * arrays the other entry points take (layout of models/cache/kvcomp_encode.py:15-67), the decode tables from
 * kvc_build_lut, the encoder's size hints (0 = unknown), `tokens` compressed tokens (a multiple of 64 for K,
 * 128 for V) and `tail_tokens` fp16 tokens [tail, batch, kv_heads, head_dim] that follow them.
 * d_workspace: kvc_attention_workspace_bytes(...) bytes of device memory, 256-byte aligned, contents ignored.
 * d_out_f32: fp32 [batch, q_heads, head_dim].
 * fused_kernel_ms (may be NULL): receives the durations of the fused K and fused V kernels; asking for them
 * makes the call wait for each of the two kernels. */
typedef struct kvc_compressed_desc {
    const void *d_luts;
    int64_t rows_per_codebook;
    const uint8_t *d_block_infos;
    int64_t block_infos_bytes;
    const uint8_t *d_thread_infos;
    int64_t thread_infos_bytes;
    const uint8_t *d_encoded;
    int64_t encoded_bytes;
    const int8_t *d_quant_min_ints;
    const void *d_quant_scales_f16;
    int64_t quant_mask;
    int64_t max_tile_bytes;
    int64_t max_stream_bytes;
    int64_t max_code_bits;
    int64_t tokens;
    const void *d_tail_f16;
    int64_t tail_tokens;
} kvc_compressed_desc;
int64_t kvc_attention_workspace_bytes(int64_t total_tokens, int64_t v_compressed_tokens, int64_t batch,
                                      int64_t q_heads, int64_t head_dim);
int kvc_attention_decode(const kvc_compressed_desc *k, const kvc_compressed_desc *v, const void *d_q_f16,
                         float softmax_scale, void *d_workspace, int64_t workspace_bytes, float *d_out_f32,
                         int64_t batch, int64_t kv_heads, int64_t q_heads, int64_t head_dim,
                         float *elapsed_ms, float *fused_kernel_ms, void *stream);

/* ---- decode attention without any allocation (no counterpart in the reference; for callers that cannot
 * allocate device memory: code under HIP graph capture, serving loops with a fixed memory plan, harnesses that
 * forbid hipMalloc) --------------------------------------------------------------------------------------------
 * kvc_attention_decode with the workspace kept in a device array of the library itself
 * (KVC_ATTENTION_STATIC_SCRATCH_BYTES per GPU the library runs on, held until the process ends) instead of a
 * caller's buffer; same arguments otherwise, no timing outputs, same results bit for bit.  Shapes whose workspace
 * (kvc_attention_workspace_bytes) exceeds the array are rejected with an error.  The call itself allocates
 * nothing and frees nothing.  The first call on a device looks the array's address up (make that call outside
 * graph capture).  Calls that overlap in time on one device share the array and race: keep them on one stream
 * or order them. */
#define KVC_ATTENTION_STATIC_SCRATCH_BYTES (40 * 1024 * 1024)
int kvc_attention_decode_static(const kvc_compressed_desc *k, const kvc_compressed_desc *v, const void *d_q_f16,
                                float softmax_scale, float *d_out_f32, int64_t batch, int64_t kv_heads,
                                int64_t q_heads, int64_t head_dim, void *stream);

/* ---- dense baseline: k_mat_vec_mul_cuda_export (kernels.cu:1182-1273) ------------------------------
 * d_k fp16 [tokens, batch, heads, head_dim], d_q fp16 [batch, heads, head_dim],
 * d_out fp16 [tokens, batch, heads].  (The reference requires batch == 1 and head_dim == 128.) */
int kvc_k_mat_vec_mul(const void *d_k_f16, const void *d_q_f16, void *d_out_f16,
                      int64_t tokens, int64_t batch, int64_t heads, int64_t head_dim,
                      float *elapsed_ms, void *stream);

/* ---- quantizer: quant (utils/compute.py:93-106; src/compute.cpp:40-58) and quant_ints (:74-91) -----
 * d_x fp16 [NB, BS, B, H, D]; groups given by quant_mask.  Bit-exact with the reference's chain of
 * fp16 PyTorch ops: scale = RN16(f32(RN16(max-min)) * eb); min_i = rint(RN16(min/scale));
 * sym = RN16(rint(RN16(x/scale)) - min_i).  Outputs: d_sym uint8 (same shape), d_min_i8 int8[groups],
 * d_scale_f16 fp16[groups] (the casts of models/cache/kvcomp_encode.py:97-98); optional fp16 copies
 * d_min_f16 (may be NULL).  Optionally accumulates the 256-bin symbol histogram into d_counts
 * (int64[256], may be NULL). */
int64_t kvc_quant_groups(int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask);
int kvc_quant(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
              float eb, uint8_t *d_sym, int8_t *d_min_i8, void *d_scale_f16, void *d_min_f16,
              int64_t *d_counts, void *stream);

/* ---- simulated quantization: quant_error (utils/compute.py:108-133), the value the reference's model caches
 * keep (models/cache/kvcomp_quant.py:51-69): quant_ints followed by (quant_int + min_quant) * quant_scale,
 * every step an fp16 tensor op on un-cast fp16 symbols and minima (so minima outside int8 do not wrap).
 * d_xhat_f16 fp16, same shape and grouping rules as kvc_quant; nothing else is written. */
int kvc_quant_error(const void *d_x_f16, int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                    float eb, void *d_xhat_f16, void *stream);

/* ---- dequantizer: (sym + min_i) * scale (models/cache/kvcomp_encode.py:146,161) --------------------
 * d_out fp16 = RN16(f32(sym + min_i) * f32(scale)), same shape as d_sym. */
int kvc_dequant(const uint8_t *d_sym, const int8_t *d_min_i8, const void *d_scale_f16,
                int64_t NB, int64_t BS, int64_t B, int64_t H, int64_t D, int quant_mask,
                void *d_out_f16, void *stream);

/* ---- whole-tensor Huffman coder: huffman_encode (utils/huffman.py:15-95) ------------------------------
 * kvc_h2_codes: 256 symbol counts -> per-symbol (code, length), the reference's construction (min-heap on
 *   frequency only, first pop = left = '0'; a lone symbol gets the one-bit code '0', utils/huffman.py:42-44).
 * kvc_h2_encode: d_sym uint8[n] (the flattened tensor, values already shifted into 0..255) -> d_bits, one byte
 *   (0 / 1) per code bit in stream order, each code most significant bit first; *h_total_bits receives the
 *   stream length.  d_bits == NULL only measures (the reference's callers use the length alone,
 *   accuracy/cr_estimate.py:46-58).  d_scratch: kvc_h2_scratch_bytes(n) bytes, 8-byte aligned.  Synchronises
 *   the stream to read the length back. */
int kvc_h2_codes(const int64_t *h_counts256, uint32_t *h_code256, uint32_t *h_length256);
int64_t kvc_h2_scratch_bytes(int64_t n);
int kvc_h2_encode(const uint8_t *d_sym, int64_t n, const uint32_t *h_code256, const uint32_t *h_length256,
                  uint8_t *d_bits, int64_t bits_cap, void *d_scratch, int64_t scratch_bytes,
                  int64_t *h_total_bits, void *stream);

/* ---- measurement aid (no counterpart in the reference) ----------------------------------------------
 * Plain device-to-device copy of `bytes` bytes (a multiple of 16) by a grid-stride kernel named
 * kvc_calibration_copy_kernel: a dispatch of exactly known HBM traffic to scale profiler counters by. */
int kvc_calibration_copy(void *d_dst, const void *d_src, int64_t bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KVCOMP_HIP_H */
