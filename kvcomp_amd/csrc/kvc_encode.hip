// kvc_encode.hip -- bit-packed Huffman tile encoder.
//
// Replaces huffman_encode / v_huffman_encode and their launchers
// (kvcomp_cuda_extension/src/kernels.cu:181-235, 419-596, 919-1011).  One wave64 per tile, lane t owns
// vector t, as one 64-thread block does in the reference.  The launches:
//
//   count  every lane adds up the code lengths of its vector; a wave prefix scan turns the 64 byte
//          counts into thread_infos and the tile's byte_num           (kernels.cu:448-465, 472-478)
//   scan   payload bytes per 1024 tiles, then every workgroup turns the byte_nums of its own 1024 tiles
//          into offsets, in tile order, without waiting for another workgroup (the reference claims
//          offsets with a global atomic in arrival order, kernels.cu:474, which makes its stream
//          layout differ from run to run)
//   emit   every lane packs its codes MSB-first straight at its final position inside an LDS image
//          of the tile payload (words it shares with a neighbour lane are merged with LDS atomic OR;
//          four codes of at most 8 bits are joined before they enter the lane's 64-bit accumulator),
//          and the wave copies the image out with aligned dword stores        (kernels.cu:181-235, 483-488)
//
// The symbols are read twice (1 B/symbol each) instead of once, which buys deterministic output
// and no per-lane scratch area: a lane's stream may be as long as the code allows.
//
// kvc_store_fused runs the same count / scan / emit sequence straight from the fp16 cache: both passes
// read the fp16 tile, quantize it (utils/compute.py:74-106, bit for bit) into an LDS tile of symbols and
// hand each lane its vector from there, so the uint8 symbol tensor never exists in HBM (the reference
// materialises it and several fp16 temporaries, models/cache/kvcomp_encode.py:86-98).
#include "kvc_common.h"
#include "kvc_quant_math.h"

struct KvcEncodeArgs {
    const uint8_t *sym;        // [tokens, stride]
    int64_t stride;
    int cols;                  // tiles per tile row
    int64_t tiles;
    int vec_len;               // symbols per vector (K: head_dim, V: 128)
    int is_k;
    const uint8_t *table;      // {u32 code; u32 length} per symbol
    int table_entries;
    uint8_t *block_infos;
    uint16_t *thread_infos;
    uint8_t *encoded;
    int64_t encoded_cap;
    uint32_t base_global_offset;   // what block_info.offset exceeds the position inside `encoded` by
    uint32_t *status;          // [0] total payload bytes, [1] error bits, [2] largest tile payload, [3] largest lane stream,
                               // [KVC_ENC_ST_BASE] block_info.offset of this call's first tile; from word
                               // KVC_ENC_STATUS_WORDS on: payload bytes of tiles 1024 j .. 1024 j + 1023
    uint32_t *idx_offset;      // {tiles, bytes}  (include/kernels.h:34-42); may be NULL
    // several codebooks: table of tile row r = table + (r / rows_per_codebook) * table_stride (0: one table for all)
    int64_t table_stride;
    int rows_per_codebook;
    const int32_t *codebook_meta;  // NULL, or int32[n_codebooks][4] from kvc_build_codebook_device (status in [3])
    int n_codebooks;
    // results left on the device (kvc_encode_async): see kvc_encode_job in include/kvcomp_hip.h
    uint32_t *stream_bytes;    // NULL, or in / out: payload bytes already in `encoded`; this call appends behind them
    uint32_t *result;          // NULL, or uint32[8]
    // one pass only: how often a wave may find a word of its look-back not ready before it gives up, and whether the
    // call is to be treated as if a wave had given up (both from the option "encode_lookback_polls")
    int max_polls, force_order;
};

constexpr int KVC_ENC_STATUS_WORDS = 16;            // status words in front of the per-1024-tile payload totals
constexpr int KVC_ENC_ST_BASE = 5;
constexpr uint32_t KVC_ENC_ERR_TILE_TOO_BIG = 1u;   // a tile payload exceeds 8191 bytes
constexpr uint32_t KVC_ENC_ERR_NO_CODE = 2u;        // a symbol without a code (length 0 or outside the table)
constexpr uint32_t KVC_ENC_ERR_CAPACITY = 4u;       // payload does not fit encoded_cap
constexpr uint32_t KVC_ENC_ERR_CODEBOOK = 8u;       // a codebook was not built (status of kvc_build_codebook_device)

// Table of the codebook that tile row `row` is encoded with.
__device__ __forceinline__ const uint8_t *kvc_table_of_row(const KvcEncodeArgs &a, int64_t row)
{
    return a.rows_per_codebook ? a.table + (row / a.rows_per_codebook) * a.table_stride : a.table;
}

// First launch of an encode call: clears the status words (a kernel, not a memset, so that the call can be recorded
// in a HIP graph), fixes the block_info.offset of the first tile (from the device counter when there is one) and
// checks that every codebook was built.
__global__ void __launch_bounds__(KVC_WAVE) kvc_encode_init_kernel(KvcEncodeArgs a)
{
    __shared__ uint32_t s_bad;
    const int tid = threadIdx.x;
    if (tid == 0) s_bad = 0;
    __syncthreads();
    if (a.codebook_meta)
        for (int i = tid; i < a.n_codebooks; i += KVC_WAVE)
            if (a.codebook_meta[4 * i + 3] != 0) atomicOr(&s_bad, KVC_ENC_ERR_CODEBOOK);
    __syncthreads();
    if (tid < KVC_ENC_STATUS_WORDS) {
        uint32_t v = 0;
        if (tid == 1) v = s_bad;
        if (tid == KVC_ENC_ST_BASE) v = a.base_global_offset + (a.stream_bytes ? *a.stream_bytes : 0u);
        a.status[tid] = v;
    }
}

// Last launch: hands the call's outcome to the caller's device words (see kvc_encode_job).
__global__ void kvc_encode_publish_kernel(KvcEncodeArgs a)
{
    const uint32_t total = a.status[0], err = a.status[1];
    if (a.result) {
        a.result[0] = total;
        a.result[1] |= err;
        if (a.status[2] > a.result[2]) a.result[2] = a.status[2];
        if (a.status[3] > a.result[3]) a.result[3] = a.status[3];
        a.result[4] += (uint32_t)a.tiles;
        a.result[5] = a.status[KVC_ENC_ST_BASE];
        if (a.status[6] > a.result[6]) a.result[6] = a.status[6];
    }
    if (a.stream_bytes && !err) *a.stream_bytes = a.status[KVC_ENC_ST_BASE] - a.base_global_offset + total;
}

// The 128 (or fewer) symbols of this lane's vector, 4 per register in stream order.
//   K: token 64*row + lane, channels vec_len*col ..          (kernels.cu:439-444: one contiguous run)
//   V: channel 64*col + lane, tokens 128*row ..              (kernels.cu:514-519: one byte per token row)
__device__ __forceinline__ void kvc_load_vector(const KvcEncodeArgs &a, int64_t tile, int lane, uint32_t v[32])
{
    const int64_t row = tile / a.cols, col = tile - row * a.cols;
    if (a.is_k) {
        const uint8_t *p = a.sym + (row * KVC_WAVE + lane) * a.stride + col * a.vec_len;
        const int nd = a.vec_len >> 2;
#pragma unroll
        for (int j = 0; j < 32; j++) v[j] = j < nd ? reinterpret_cast<const uint32_t *>(p)[j] : 0u;
    } else {
        const uint8_t *p = a.sym + row * KVC_V_TOKENS * a.stride + col * KVC_WAVE + lane;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            uint32_t w = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) w |= (uint32_t)p[(int64_t)(4 * j + k) * a.stride] << (8 * k);
            v[j] = w;
        }
    }
}

// LDS traffic between the lanes of one wave needs no workgroup barrier (a wave's LDS operations complete in
// order); this keeps the compiler from moving accesses across the hand-over.
__device__ __forceinline__ void kvc_wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// A tile's symbols change hands between lanes through a staging area in LDS (the lane that loads or quantizes a symbol
// is not the lane whose vector it belongs to).  The area holds a part of the tile at a time -- half of it, or a quarter
// where V is quantized from fp16 -- so that, in the one-pass kernel, a payload of any size (up to KVC_MAX_TILE_BYTES)
// can wait in the same wave's LDS while the next tile is staged.
constexpr int KVC_STAGE_K_BYTES = 32 * (128 + 4);       // 32 tokens of up to 128 symbols, rows 4 bytes apart from a multiple of 128 (from
                                                        // symbols: also 48 tokens of at most 80 symbols, 64 of at most 64)
constexpr int KVC_STAGE_VSYM_BYTES = 64 * (64 + 4);     // 64 channels of 64 tokens
constexpr int KVC_STAGE_VF16_BYTES = 64 * (32 + 4);     // 64 channels of 32 tokens

// The same vectors of a V tile fetched four channels per lane: 16 lanes cover a token's 64 symbols, a load instruction
// four tokens (the byte-per-token-row loads above move 64 bytes per instruction, 128 instructions per tile; these move
// 256 bytes, 32 instructions), four tokens of four channels are transposed in registers and go to the staging area
// as [channel][token], 64 tokens at a time, and lane c then reads channel c's vector.  Needs the row stride to be a
// multiple of 4 and the symbols 4-byte aligned (every encode call is checked for that).
__device__ __forceinline__ void kvc_load_vector_v_tile(const KvcEncodeArgs &a, int64_t tile, int lane, uint8_t *s_stage, uint32_t v[32])
{
    constexpr int RS = 64 + 4;
    const int64_t row = tile / a.cols, col = tile - row * a.cols;
    const int pr = lane & 15, sub = lane >> 4;
    const uint8_t *p = a.sym + (row * KVC_V_TOKENS + 4 * sub) * a.stride + col * KVC_WAVE + 4 * pr;
    uint32_t w[32];
#pragma unroll
    for (int jj = 0; jj < 8; jj++)
#pragma unroll
        for (int k = 0; k < 4; k++) w[4 * jj + k] = *reinterpret_cast<const uint32_t *>(p + (int64_t)(16 * jj + k) * a.stride);
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int jj = 4 * h; jj < 4 * h + 4; jj++) {
            const uint32_t w0 = w[4 * jj], w1 = w[4 * jj + 1], w2 = w[4 * jj + 2], w3 = w[4 * jj + 3];
            // {w0.b0 w1.b0 w0.b1 w1.b1}, {w0.b2 w1.b2 w0.b3 w1.b3}, the same of w2 and w3; then a channel's four tokens
            const uint32_t a_lo = __builtin_amdgcn_perm(w1, w0, 0x05010400u), a_hi = __builtin_amdgcn_perm(w1, w0, 0x07030602u);
            const uint32_t b_lo = __builtin_amdgcn_perm(w3, w2, 0x05010400u), b_hi = __builtin_amdgcn_perm(w3, w2, 0x07030602u);
            const uint32_t c0 = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u), c1 = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
            const uint32_t c2 = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u), c3 = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
            uint8_t *dst = s_stage + (4 * pr) * RS + 16 * (jj - 4 * h) + 4 * sub;
            *reinterpret_cast<uint32_t *>(dst) = c0;
            *reinterpret_cast<uint32_t *>(dst + RS) = c1;
            *reinterpret_cast<uint32_t *>(dst + 2 * RS) = c2;
            *reinterpret_cast<uint32_t *>(dst + 3 * RS) = c3;
        }
        kvc_wave_lds_sync();
#pragma unroll
        for (int j = 0; j < 16; j++) v[16 * h + j] = *reinterpret_cast<const uint32_t *>(s_stage + lane * RS + 4 * j);
        kvc_wave_lds_sync();                                           // read: the area may take the next part
    }
}

// Token `lane`'s row of a K staging area that holds tokens 32 h .. 32 h + 31 (rows RS bytes apart).
__device__ __forceinline__ void kvc_read_k_rows(const uint8_t *s_stage, int RS, int nd, int lane, int h, uint32_t (&v)[32])
{
    if ((lane >> 5) == h) {
        const uint8_t *row = s_stage + (lane & 31) * RS;
#pragma unroll
        for (int j = 0; j < 32; j++)
            if (j < nd) v[j] = *reinterpret_cast<const uint32_t *>(row + 4 * j);
    }
}

// K vectors through the staging area as well: vec_len / 4 lanes cover a token's run, a load instruction two or more tokens
// (with a token per lane, as above, every instruction touches 64 rows of the symbol tensor), the words go to the area
// as [token][channel] with rows vec_len + 4 bytes apart, 32 tokens at a time, and lane t then reads token t's row.
// vec_len <= 128.
__device__ __forceinline__ void kvc_load_vector_k_tile(const KvcEncodeArgs &a, int64_t tile, int lane, uint8_t *s_stage, uint32_t (&v)[32])
{
    const int64_t row = tile / a.cols, col = tile - row * a.cols;
    const int nd = a.vec_len >> 2, RS = a.vec_len + 4;
    const int per = KVC_WAVE / nd;                                     // tokens per load instruction (at least 2)
    const int r = lane / nd, cw = lane - r * nd;
    const bool active = r < per;
    const uint8_t *p = a.sym + (row * KVC_WAVE + r) * a.stride + col * a.vec_len + 4 * cw;
    uint32_t w[32];
#pragma unroll
    for (int i = 0; i < 32; i++) {
        w[i] = 0u;
        if (active && r + per * i < KVC_WAVE) w[i] = *reinterpret_cast<const uint32_t *>(p + (int64_t)(per * i) * a.stride);
    }
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = 0u;
    // the first sixteen load instructions cover tokens 0 .. 16 per - 1 (all 64 where a token's run is at most 64 bytes),
    // the other sixteen the rest: at most 32 tokens of 132 bytes, 48 of 84 or 64 of 68 in the area at a time
    const int split = 16 * per;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        uint8_t *dst = s_stage + r * RS + 4 * cw;
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (active && r + per * (16 * h + i) < KVC_WAVE) *reinterpret_cast<uint32_t *>(dst + (per * i) * RS) = w[16 * h + i];
        kvc_wave_lds_sync();
        const int mine = lane - split * h;                 // this lane's row of the area, if it is in this part
        if (mine >= 0 && (h == 1 || mine < split)) {
            const uint8_t *rowp = s_stage + mine * RS;
#pragma unroll
            for (int j = 0; j < 32; j++)
                if (j < nd) v[j] = *reinterpret_cast<const uint32_t *>(rowp + 4 * j);
        }
        kvc_wave_lds_sync();
    }
}

// What the count step of one tile finds out (every field wave-uniform except `start`).
struct KvcTileCount {
    uint32_t start;      // first byte of this lane's stream inside the tile payload
    uint32_t bytes;      // payload bytes of the tile
    uint32_t longest;    // longest lane stream of the tile
    uint32_t err;        // error bits raised by any lane
};

// Count step for one tile: adds up the code lengths of the lane's vector, writes the 64 thread_infos.
__device__ __forceinline__ KvcTileCount kvc_count_vectors(const KvcEncodeArgs &a, int64_t tile, int lane, const uint32_t (&v)[32],
                                                          const uint8_t *s_len)
{
    uint32_t bits = 0, bad = 0;
    const int nd = a.vec_len >> 2;
#pragma unroll
    for (int j = 0; j < 32; j++) {
        if (j < nd) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t l = s_len[(v[j] >> (8 * k)) & 0xffu];
                bits += l;
                bad |= (l == 0);
            }
        }
    }
    const uint32_t bytes = (bits + 7u) >> 3;
    const uint32_t end = kvc_wave_inclusive_scan(bytes, lane);
    a.thread_infos[tile * KVC_WAVE + lane] = (uint16_t)((end << 3) + (bytes << 3) - bits);
    KvcTileCount c;
    c.start = end - bytes;
    c.bytes = (uint32_t)__builtin_amdgcn_readlane((int)end, KVC_WAVE - 1);
    c.err = __any(bad) ? KVC_ENC_ERR_NO_CODE : 0u;
    if (c.bytes > (uint32_t)KVC_MAX_TILE_BYTES) c.err |= KVC_ENC_ERR_TILE_TOO_BIG;
    uint32_t longest = bytes;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)longest, off, 64);
        longest = o > longest ? o : longest;
    }
    c.longest = longest;
    return c;
}

// Count pass for one tile: thread_infos, byte_num, error bits; returns the lane-stream maximum of the wave.
__device__ __forceinline__ uint32_t kvc_count_tile(const KvcEncodeArgs &a, int64_t tile, int lane, const uint32_t (&v)[32],
                                                   const uint8_t *s_len, uint32_t *s_err)
{
    const KvcTileCount c = kvc_count_vectors(a, tile, lane, v, s_len);
    // byte_num; the offset half of block_info is filled in by the scan kernel
    if (lane == KVC_WAVE - 1) reinterpret_cast<uint32_t *>(a.block_infos + 8 * tile)[1] = c.bytes > 0xffffu ? 0xffffu : c.bytes;
    if (c.err && lane == 0) atomicOr(s_err, c.err);
    return c.longest;
}

// Code lengths of the table that `tile` is encoded with, one copy per wave (the tiles of a workgroup may lie in
// rows with different codebooks).
__device__ __forceinline__ void kvc_load_len_table(const KvcEncodeArgs &a, int64_t tile, uint8_t *s_len, int lane)
{
    const uint32_t *t = reinterpret_cast<const uint32_t *>(kvc_table_of_row(a, tile / a.cols));
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int i = lane + KVC_WAVE * k;
        uint32_t len = 0;
        if (i < a.table_entries) len = t[2 * i + 1];
        s_len[i] = (uint8_t)(len > 32 ? 0 : len);
    }
}

__global__ void __launch_bounds__(KVC_WG) kvc_encode_count_kernel(KvcEncodeArgs a)
{
    __shared__ uint8_t s_len[KVC_WAVES_PER_WG][256];
    __shared__ uint32_t s_err, s_longest;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) { s_err = 0; s_longest = 0; }
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (tile < a.tiles) kvc_load_len_table(a, tile, s_len[wave], lane);
    __syncthreads();
    if (tile < a.tiles) {
        uint32_t v[32];
        kvc_load_vector(a, tile, lane, v);
        const uint32_t longest = kvc_count_tile(a, tile, lane, v, s_len[wave], &s_err);
        if (lane == 0) atomicMax(&s_longest, longest);
    }
    __syncthreads();
    if (tid == 0 && s_err) atomicOr(&a.status[1], s_err);
    if (tid == 0) atomicMax(&a.status[3], s_longest);
}

// Payload bytes of tiles [1024 c, 1024 c + 1024), one workgroup per c.
__global__ void __launch_bounds__(1024) kvc_encode_chunk_sum_kernel(KvcEncodeArgs a)
{
    __shared__ uint32_t s_wave[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile = (int64_t)blockIdx.x * 1024 + tid;
    uint32_t bn = 0;
    if (tile < a.tiles) bn = reinterpret_cast<const uint32_t *>(a.block_infos + 8 * tile)[1] & 0xffffu;
    const uint32_t incl = kvc_wave_inclusive_scan(bn, lane);
    if (lane == KVC_WAVE - 1) s_wave[wave] = incl;
    __syncthreads();
    if (tid == 0) {
        uint32_t total = 0;
        for (int w = 0; w < 16; w++) total += s_wave[w];
        a.status[KVC_ENC_STATUS_WORDS + blockIdx.x] = total;
    }
}

// Workgroup c turns the byte_nums of tiles [1024 c, 1024 c + 1024) into offsets: what lies in front of its
// range is the sum of the per-1024-tile totals of the kernel above, the rest is a scan of its own 1024
// values.  No workgroup waits for another.
__global__ void __launch_bounds__(1024) kvc_encode_scan_kernel(KvcEncodeArgs a)
{
    __shared__ uint32_t s_wave[16], s_before[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t *chunk_sums = a.status + KVC_ENC_STATUS_WORDS;
    const int64_t chunks = (a.tiles + 1023) / 1024;
    uint32_t part = 0;
    for (int64_t j = tid; j < chunks; j += 1024) part += j < (int64_t)blockIdx.x ? chunk_sums[j] : 0u;
    uint32_t all = 0;
    if (blockIdx.x == 0) for (int64_t j = tid; j < chunks; j += 1024) all += chunk_sums[j];
    const int64_t tile = (int64_t)blockIdx.x * 1024 + tid;
    uint32_t bn = 0;
    if (tile < a.tiles) bn = reinterpret_cast<const uint32_t *>(a.block_infos + 8 * tile)[1] & 0xffffu;
    const uint32_t incl = kvc_wave_inclusive_scan(bn, lane);
    const uint32_t part_w = kvc_wave_inclusive_scan(part, lane);
    uint32_t mx = bn;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)mx, off, 64);
        mx = o > mx ? o : mx;
    }
    if (lane == KVC_WAVE - 1) {
        s_wave[wave] = incl;
        s_before[wave] = part_w;
    }
    if (lane == 0 && mx) atomicMax(&a.status[2], mx);
    __syncthreads();
    uint32_t before = a.status[KVC_ENC_ST_BASE];
    for (int w = 0; w < 16; w++) {
        before += s_before[w];
        if (w < wave) before += s_wave[w];
    }
    if (tile < a.tiles) reinterpret_cast<uint32_t *>(a.block_infos + 8 * tile)[0] = before + incl - bn;
    if (blockIdx.x == 0) {
        // the grand total, by the first workgroup
        const uint32_t all_w = kvc_wave_inclusive_scan(all, lane);
        __syncthreads();
        if (lane == KVC_WAVE - 1) s_before[wave] = all_w;
        __syncthreads();
        if (tid == 0) {
            uint32_t total = 0;
            for (int w = 0; w < 16; w++) total += s_before[w];
            a.status[0] = total;
            const int64_t first = (int64_t)a.status[KVC_ENC_ST_BASE] - a.base_global_offset;      // position inside `encoded`
            if (first + total > a.encoded_cap) atomicOr(&a.status[1], KVC_ENC_ERR_CAPACITY);
            if (a.idx_offset) {
                a.idx_offset[0] = (uint32_t)a.tiles;
                a.idx_offset[1] = total;
            }
        }
    }
}

constexpr int KVC_IMAGE_WORDS = (KVC_MAX_TILE_BYTES + 3 + 3) / 4 + 1;   // payload + up to 3 leading bytes

// Where tile `tile` goes: ok = it fits (a tile flagged by the earlier launches is skipped, never written out of bounds).
struct KvcEmitPlace {
    uint32_t off, bn, head;
    bool ok;
};

__device__ __forceinline__ KvcEmitPlace kvc_emit_place(const KvcEncodeArgs &a, int64_t tile, bool active)
{
    KvcEmitPlace p = {0u, 0u, 0u, false};
    if (active) {
        const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.block_infos + 8 * tile);
        p.off = bi[0] - a.base_global_offset;
        p.bn = bi[1] & 0xffffu;
    }
    p.ok = active && p.bn <= (uint32_t)KVC_MAX_TILE_BYTES && (int64_t)p.off + p.bn <= a.encoded_cap;
    if (p.ok) p.head = (uint32_t)((reinterpret_cast<uintptr_t>(a.encoded) + p.off) & 3u);
    return p;
}

// A wave's copy of the encode table of its tile: entries without a usable code become {0, 0} (the count pass has
// flagged them), and *s_short tells whether every code has at most 8 bits (four then fit one 32-bit group).
// The caller initialises *s_short (the wave's own word) to 1 and synchronises before and after.
__device__ __forceinline__ void kvc_load_code_table(const KvcEncodeArgs &a, int64_t tile, uint2 *s_table, uint32_t *s_short, int lane)
{
    const uint2 *t = reinterpret_cast<const uint2 *>(kvc_table_of_row(a, tile / a.cols));
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int i = lane + KVC_WAVE * k;
        uint2 e = i < a.table_entries ? t[i] : make_uint2(0u, 0u);
        if (e.y > 32u) e = make_uint2(0u, 0u);
        if (e.y < 32u) e.x &= (1u << e.y) - 1u;           // nothing above the code's own bits
        s_table[i] = e;
        if (e.y > 8u) atomicAnd(s_short, 0u);
    }
}

// Pack this lane's vector MSB-first at its final position inside the (zeroed) LDS image of the tile payload.
// The lane's bits pass through a 64-bit accumulator; whenever it holds 32 or more, the oldest 32 leave for the
// image (what is left above the live bits is never read again, so it is not cleared).  With codes of at most
// 8 bits the four symbols of a register are first joined into one group of at most 32 bits, which costs a
// quarter of the accumulator traffic.
// Where lane `lane`'s stream starts inside the payload of `tile`, from the thread_infos an earlier launch wrote.
__device__ __forceinline__ uint32_t kvc_stream_start(const KvcEncodeArgs &a, int64_t tile, int lane)
{
    return lane ? (uint32_t)(a.thread_infos[tile * KVC_WAVE + lane - 1] >> 3) : 0u;
}

__device__ __forceinline__ void kvc_pack_vector(const KvcEncodeArgs &a, uint32_t start, const uint32_t (&v)[32],
                                                const uint2 *s_table, uint32_t *image, uint32_t head, bool short_codes,
                                                uint32_t image_words = (uint32_t)KVC_IMAGE_WORDS)
{
    const uint32_t bitpos = (head + start) * 8u;
    uint32_t w = bitpos >> 5, nacc = bitpos & 31u;
    uint64_t acc = 0;
    const int nd = a.vec_len >> 2;
    auto push = [&](uint32_t bits, uint32_t len) {       // len <= 32, nacc < 32
        acc = (acc << len) | bits;
        nacc += len;
        if (nacc >= 32u) {
            nacc -= 32u;
            if (w < image_words) atomicOr(&image[w], kvc_bswap((uint32_t)(acc >> nacc)));
            w++;
        }
    };
    if (short_codes) {                                   // wave-uniform
#pragma unroll
        for (int j = 0; j < 32; j++) {
            if (j < nd) {
                const uint2 e0 = s_table[v[j] & 0xffu], e1 = s_table[(v[j] >> 8) & 0xffu];
                const uint2 e2 = s_table[(v[j] >> 16) & 0xffu], e3 = s_table[v[j] >> 24];
                const uint32_t g = ((((e0.x << e1.y) | e1.x) << e2.y | e2.x) << e3.y) | e3.x;
                push(g, e0.y + e1.y + e2.y + e3.y);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; j++) {
            if (j < nd) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint2 e = s_table[(v[j] >> (8 * k)) & 0xffu];
                    push(e.x, e.y);
                }
            }
        }
    }
    if (nacc > 0 && w < image_words) atomicOr(&image[w], kvc_bswap((uint32_t)(acc << (32u - nacc))));
}

// Copy the image out with aligned dword stores (bytes at the two ragged ends).
__device__ __forceinline__ void kvc_write_image(const KvcEncodeArgs &a, const KvcEmitPlace &p, int lane, const uint32_t *image)
{
    uint8_t *dst = a.encoded + p.off - p.head;                 // 4-byte aligned
    const uint32_t lo = p.head, hi = p.head + p.bn;            // valid byte range inside the image
    const uint32_t nwords = (hi + 3u) >> 2;
    for (uint32_t f = lane; f < nwords; f += KVC_WAVE) {
        const uint32_t b0 = 4u * f, word = image[f];
        if (b0 >= lo && b0 + 4u <= hi) {
            reinterpret_cast<uint32_t *>(dst)[f] = word;
        } else {
#pragma unroll
            for (uint32_t k = 0; k < 4; k++)
                if (b0 + k >= lo && b0 + k < hi) dst[b0 + k] = (uint8_t)(word >> (8u * k));
        }
    }
}

// The same for an image that was packed from its first word on, while the payload starts p.head bytes into an
// aligned word of the destination: every output word is put together from two image words.
__device__ __forceinline__ void kvc_write_image_shifted(const KvcEncodeArgs &a, const KvcEmitPlace &p, int lane, const uint32_t *image)
{
    uint8_t *dst = a.encoded + p.off - p.head;                 // 4-byte aligned
    const uint32_t lo = p.head, hi = p.head + p.bn;            // valid byte range of the output words
    const uint32_t nwords = (hi + 3u) >> 2;
    const uint32_t shift = 8u * (4u - p.head);                 // 32, 24, 16, 8
    for (uint32_t f = lane; f < nwords; f += KVC_WAVE) {
        const uint32_t cur = f < (uint32_t)KVC_IMAGE_WORDS ? image[f] : 0u, prev = f ? image[f - 1] : 0u;
        const uint32_t b0 = 4u * f, word = (uint32_t)((((uint64_t)cur << 32) | prev) >> shift);
        if (b0 >= lo && b0 + 4u <= hi) {
            reinterpret_cast<uint32_t *>(dst)[f] = word;
        } else {
#pragma unroll
            for (uint32_t k = 0; k < 4; k++)
                if (b0 + k >= lo && b0 + k < hi) dst[b0 + k] = (uint8_t)(word >> (8u * k));
        }
    }
}

__global__ void __launch_bounds__(KVC_WG) kvc_encode_emit_kernel(KvcEncodeArgs a)
{
    __shared__ uint2 s_table[KVC_WAVES_PER_WG][256];
    __shared__ uint32_t s_short[KVC_WAVES_PER_WG];
    __shared__ uint32_t s_image[KVC_WAVES_PER_WG][KVC_IMAGE_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (lane == 0) s_short[wave] = 1u;
    __syncthreads();
    if (tile < a.tiles) kvc_load_code_table(a, tile, s_table[wave], &s_short[wave], lane);
    uint32_t *image = s_image[wave];
    __syncthreads();
    const KvcEmitPlace p = kvc_emit_place(a, tile, tile < a.tiles);
    if (!p.ok) return;                                 // wave-uniform; each wave has its own image from here on
    const uint32_t image_words = (p.head + p.bn + 3u) / 4u + 1u;
    for (uint32_t i = lane; i < image_words && i < (uint32_t)KVC_IMAGE_WORDS; i += KVC_WAVE) image[i] = 0;
    uint32_t v[32];
    kvc_load_vector(a, tile, lane, v);
    kvc_wave_lds_sync();
    kvc_pack_vector(a, kvc_stream_start(a, tile, lane), v, s_table[wave], image, p.head, s_short[wave] != 0u);
    kvc_wave_lds_sync();
    kvc_write_image(a, p, lane, image);
}

// ---------------------------------------------------------------------------------------------------
// fused quantize + encode: the front end that turns an fp16 tile into this lane's vector of symbols
// ---------------------------------------------------------------------------------------------------
struct KvcStoreArgs {
    KvcEncodeArgs e;           // e.sym is unused
    const __half *x;           // [tokens, stride] fp16
    int B, H, D;               // stride = B * H * D
    int mask;                  // quantization groups (KVC_MASK_*)
    float eb;
    int8_t *min_i8;            // per-channel K: written by the count pass; every other layout: read (written by
    __half *scale_f16;         // the parameter pass that runs first)
};

constexpr int KVC_SYM_TILE_BYTES = 64 * (128 + 4);      // 64 vectors of up to 128 symbols, rows 4 bytes apart from a multiple of 128
static_assert(KVC_SYM_TILE_BYTES >= KVC_IMAGE_WORDS * 4, "the payload image reuses the symbol tile");

__device__ __forceinline__ KvcGroupParams kvc_stored_params(const KvcStoreArgs &a, int64_t g)
{
    KvcGroupParams p;
    p.scale_h = a.scale_f16[g];
    p.scale = __half2float(p.scale_h);
    p.rcp = __fdiv_rn(1.0f, p.scale);
    p.min_i = (float)a.min_i8[g];
    p.min_h = __float2half_rn(p.min_i);
    return p;
}

// K tile: 64 tokens x D channels of one (batch, head).  Lane l owns channels 2l and 2l + 1 while the tile is
// quantized (each load instruction of the wave is one token's contiguous run of D halves), the symbols go
// to LDS as [token][channel], and lane t then reads token t's vector.
// Per-channel groups live entirely inside the tile: the count pass (kvc_front_k_once) finds min / max itself, writes
// the group parameters and quantizes with exactly what it wrote (the minimum as int8), the emit pass (kvc_front_k)
// reads them back, so the two passes always agree.  Both quantize with packed fp16 arithmetic
// (kvc_quant_pair_biased: two channels per instruction).
__device__ __forceinline__ void kvc_front_k(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, uint32_t (&v)[32])
{
    const int64_t stride = a.e.stride;
    const int D = a.D, RS = D + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const bool act = 2 * lane < D;
    const __half *p = a.x + (row * KVC_WAVE) * stride + col * D + (act ? 2 * lane : 0);
    KvcGroupParams g0, g1;
    if (a.mask == KVC_MASK_CHANNEL) {
        const int64_t g = row * stride + col * D + (act ? 2 * lane : 0);
        g0 = kvc_stored_params(a, g);
        g1 = kvc_stored_params(a, g + 1);
    } else {                                             // one pair per 64-token block (kernels.cu:771-772)
        g0 = g1 = kvc_stored_params(a, row);
    }
    const KvcPackedParams pp = kvc_packed_params(g0, g1);
    const int nd = D >> 2;
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = 0u;
#pragma unroll
    for (int h = 0; h < 2; h++) {                         // 32 tokens at a time through the staging area
        if (act) {
#pragma unroll 8
            for (int t = 0; t < 32; t++) {
                const uint32_t u = kvc_quant_pair_biased(*reinterpret_cast<const uint32_t *>(p + (32 * h + t) * stride), pp);
                *reinterpret_cast<uint16_t *>(s_sym + t * RS + 2 * lane) = (uint16_t)kvc_low_bytes4(u, u);
            }
        }
        kvc_wave_lds_sync();
        kvc_read_k_rows(s_sym, RS, nd, lane, h, v);
        kvc_wave_lds_sync();
    }
}

// The count pass's variant: the lane keeps its two channels of all 64 tokens in registers (kvc_front_k_load: 64 loads in
// flight, one walk over the tile), finds the groups' minima and maxima there (packed fp16 min / max), publishes the group
// parameters and quantizes.
__device__ __forceinline__ void kvc_front_k_load(const KvcStoreArgs &a, int64_t tile, int lane, uint32_t (&raw)[KVC_WAVE])
{
    const int64_t stride = a.e.stride;
    const int D = a.D;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const __half *p = a.x + (row * KVC_WAVE) * stride + col * D + (2 * lane < D ? 2 * lane : 0);
#pragma unroll
    for (int t = 0; t < KVC_WAVE; t++) raw[t] = *reinterpret_cast<const uint32_t *>(p + t * stride);
}

__device__ __forceinline__ void kvc_front_k_once(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, const uint32_t (&raw)[KVC_WAVE],
                                                 uint32_t (&v)[32])
{
    const int64_t stride = a.e.stride;
    const int D = a.D, RS = D + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const bool act = 2 * lane < D;
    KvcGroupParams g0, g1;
    if (a.mask == KVC_MASK_CHANNEL) {
        const int64_t g = row * stride + col * D + (act ? 2 * lane : 0);
        kvc_half2 mn = __builtin_bit_cast(kvc_half2, raw[0]), mx = mn;
#pragma unroll
        for (int t = 1; t < KVC_WAVE; t++) {
            const kvc_half2 x = __builtin_bit_cast(kvc_half2, raw[t]);
            mn = __builtin_elementwise_min(mn, x);
            mx = __builtin_elementwise_max(mx, x);
        }
        const uint32_t mnw = __builtin_bit_cast(uint32_t, mn), mxw = __builtin_bit_cast(uint32_t, mx);
        g0 = kvc_group_params(kvc_half_lo(mnw), kvc_half_lo(mxw), a.eb);
        g1 = kvc_group_params(kvc_half_hi(mnw), kvc_half_hi(mxw), a.eb);
        const int8_t m0 = (int8_t)(int)g0.min_i, m1 = (int8_t)(int)g1.min_i;     // quantize with the minimum as it is stored
        g0.min_i = (float)m0;
        g1.min_i = (float)m1;
        g0.min_h = __float2half_rn(g0.min_i);
        g1.min_h = __float2half_rn(g1.min_i);
        if (act) {
            a.scale_f16[g] = g0.scale_h;
            a.scale_f16[g + 1] = g1.scale_h;
            a.min_i8[g] = m0;
            a.min_i8[g + 1] = m1;
        }
    } else {                                             // one pair per 64-token block (kernels.cu:771-772)
        g0 = g1 = kvc_stored_params(a, row);
    }
    const KvcPackedParams pp = kvc_packed_params(g0, g1);
    const int nd = D >> 2;
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = 0u;
#pragma unroll
    for (int h = 0; h < 2; h++) {                         // 32 tokens at a time through the staging area
        if (act) {
#pragma unroll
            for (int t = 0; t < 32; t++) {
                const uint32_t u = kvc_quant_pair_biased(raw[32 * h + t], pp);
                *reinterpret_cast<uint16_t *>(s_sym + t * RS + 2 * lane) = (uint16_t)kvc_low_bytes4(u, u);
            }
        }
        kvc_wave_lds_sync();
        kvc_read_k_rows(s_sym, RS, nd, lane, h, v);
        kvc_wave_lds_sync();
    }
}

// V tile: 128 tokens x 64 flat channels.  While the tile is quantized, lane l owns channels 2 (l & 31), + 1 of
// tokens 64 (l >> 5) .. + 63 (one load instruction = two tokens' runs of 64 halves); four tokens' symbols of a
// channel are gathered in a register and written to LDS as one word of the [channel][token] tile, and lane c
// then reads channel c's vector.  Group parameters are per token (KVC_MASK_V_TOKEN) or per (token, batch
// entry) (KVC_MASK_SIM_TOKEN; the tile lies inside one batch entry); the wave first stages its 128 triples
// {scale, 1 / scale, min} in LDS.
__device__ __forceinline__ void kvc_front_v_load(const KvcStoreArgs &a, int64_t tile, int lane, uint32_t (&raw)[KVC_WAVE])
{
    const int64_t stride = a.e.stride;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const int pr = lane & 31, half = lane >> 5;
    const __half *p = a.x + (row * KVC_V_TOKENS + 64 * half) * stride + col * KVC_WAVE + 2 * pr;
#pragma unroll
    for (int t = 0; t < KVC_WAVE; t++) raw[t] = *reinterpret_cast<const uint32_t *>(p + (int64_t)t * stride);
}

// raw: the lane's channel pair of its 64 tokens, as kvc_front_v_load fetched them (all 64 loads in flight at once: taken
// four at a time between the quantizing, the loop waited for memory sixteen times)
__device__ __forceinline__ void kvc_front_v(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, uint32_t *s_par,
                                            const uint32_t (&raw)[KVC_WAVE], uint32_t (&v)[32])
{
    constexpr int RS = 32 + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const int pr = lane & 31, half = lane >> 5;
    const int64_t b = (col * KVC_WAVE) / ((int64_t)a.H * a.D);
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int t = lane + 64 * k;
        const int64_t tk = row * KVC_V_TOKENS + t;
        const KvcGroupParams g = kvc_stored_params(a, a.mask == KVC_MASK_V_TOKEN ? tk : tk * a.B + b);
        const KvcPackedParams pp = kvc_packed_params(g, g);          // the token's constants in both halves
        *reinterpret_cast<uint4 *>(s_par + 4 * t) = make_uint4(pp.P2, pp.S2, pp.r2, pp.c2);
    }
    kvc_wave_lds_sync();
#pragma unroll
    for (int q = 0; q < 4; q++) {                         // a quarter of the tile at a time: tokens 16 q .. + 15 of either half
#pragma unroll
        for (int jj = 4 * q; jj < 4 * q + 4; jj++) {
            uint32_t u[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int t = 64 * half + 4 * jj + k;
                const uint4 c = *reinterpret_cast<const uint4 *>(s_par + 4 * t);
                const KvcPackedParams pp = {c.x, c.y, c.z, c.w};
                u[k] = kvc_quant_pair_biased(raw[4 * jj + k], pp);
            }
            // a01 = {channel 2 pr, 2 pr + 1 of token 4 jj | the same of token 4 jj + 1}; then four tokens of each channel
            const uint32_t a01 = kvc_low_bytes4(u[0], u[1]), a23 = kvc_low_bytes4(u[2], u[3]);
            const uint32_t w0 = kvc_low_bytes4(a01, a23), w1 = __builtin_amdgcn_perm(a23, a01, 0x07050301u);
            *reinterpret_cast<uint32_t *>(s_sym + (2 * pr) * RS + 16 * half + 4 * (jj - 4 * q)) = w0;
            *reinterpret_cast<uint32_t *>(s_sym + (2 * pr + 1) * RS + 16 * half + 4 * (jj - 4 * q)) = w1;
        }
        kvc_wave_lds_sync();
#pragma unroll
        for (int k = 0; k < 4; k++) {                     // register j holds tokens 4 j .. 4 j + 3 of the lane's channel
            v[4 * q + k] = *reinterpret_cast<const uint32_t *>(s_sym + lane * RS + 4 * k);
            v[16 + 4 * q + k] = *reinterpret_cast<const uint32_t *>(s_sym + lane * RS + 16 + 4 * k);
        }
        kvc_wave_lds_sync();                               // read: the area may take the next quarter
    }
}

template <bool IS_K>
__global__ void __launch_bounds__(KVC_WG) kvc_store_count_kernel(KvcStoreArgs a)
{
    __shared__ uint8_t s_len[KVC_WAVES_PER_WG][256];
    __shared__ uint32_t s_err, s_longest;
    __shared__ __align__(16) uint8_t s_sym[KVC_WAVES_PER_WG][KVC_SYM_TILE_BYTES];
    __shared__ __align__(16) uint32_t s_par[IS_K ? 1 : KVC_WAVES_PER_WG][IS_K ? 4 : 4 * KVC_V_TOKENS];   // V: the packed constants of every token
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) { s_err = 0; s_longest = 0; }
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (tile < a.e.tiles) kvc_load_len_table(a.e, tile, s_len[wave], lane);
    __syncthreads();
    if (tile < a.e.tiles) {
        uint32_t v[32];
        if (IS_K) {
            uint32_t raw[KVC_WAVE];
            kvc_front_k_load(a, tile, lane, raw);
            kvc_front_k_once(a, tile, lane, s_sym[wave], raw, v);
        } else {
            uint32_t raw[KVC_WAVE];
            kvc_front_v_load(a, tile, lane, raw);
            kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], raw, v);
        }
        const uint32_t longest = kvc_count_tile(a.e, tile, lane, v, s_len[wave], &s_err);
        if (lane == 0) atomicMax(&s_longest, longest);
    }
    __syncthreads();
    if (tid == 0 && s_err) atomicOr(&a.e.status[1], s_err);
    if (tid == 0) atomicMax(&a.e.status[3], s_longest);
}

template <bool IS_K>
__global__ void __launch_bounds__(KVC_WG) kvc_store_emit_kernel(KvcStoreArgs a)
{
    __shared__ uint2 s_table[KVC_WAVES_PER_WG][256];
    __shared__ __align__(16) uint8_t s_sym[KVC_WAVES_PER_WG][KVC_SYM_TILE_BYTES];   // symbols first, then the payload image
    __shared__ __align__(16) uint32_t s_par[IS_K ? 1 : KVC_WAVES_PER_WG][IS_K ? 4 : 4 * KVC_V_TOKENS];
    __shared__ uint32_t s_short[KVC_WAVES_PER_WG];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (lane == 0) s_short[wave] = 1u;
    __syncthreads();
    if (tile < a.e.tiles) kvc_load_code_table(a.e, tile, s_table[wave], &s_short[wave], lane);
    __syncthreads();
    const KvcEmitPlace p = kvc_emit_place(a.e, tile, tile < a.e.tiles);
    if (!p.ok) return;                                 // wave-uniform; nothing below involves another wave
    uint32_t *image = reinterpret_cast<uint32_t *>(s_sym[wave]);
    uint32_t v[32];
    if (IS_K) {
        kvc_front_k(a, tile, lane, s_sym[wave], v);
    } else {
        uint32_t raw[KVC_WAVE];
        kvc_front_v_load(a, tile, lane, raw);
        kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], raw, v);
    }
    kvc_wave_lds_sync();                               // every lane holds its vector: the tile can be overwritten
    const uint32_t image_words = (p.head + p.bn + 3u) / 4u + 1u;
    for (uint32_t i = lane; i < image_words && i < (uint32_t)KVC_IMAGE_WORDS; i += KVC_WAVE) image[i] = 0;
    kvc_wave_lds_sync();
    kvc_pack_vector(a.e, kvc_stream_start(a.e, tile, lane), v, s_table[wave], image, p.head, s_short[wave] != 0u);
    kvc_wave_lds_sync();
    kvc_write_image(a.e, p, lane, image);
}

// ---------------------------------------------------------------------------------------------------
// one pass: count, place and emit a tile in the same wave
// ---------------------------------------------------------------------------------------------------
// The two-pass encoder reads (and, in the fused store, quantizes) every tile twice and looks every symbol up twice,
// because a tile's position in the payload is the sum of the sizes of all tiles before it.  Here a wave keeps its tile:
// it looks its symbols up once (four codes of at most 8 bits joined into one group, the groups kept in the registers
// that held the symbols), publishes the tile's size, finds its offset by looking back over the tiles before it
// (decoupled look-back), and packs and writes the payload.  The offsets are the same exact prefix sums in tile order,
// so the output is byte for byte that of the two-pass encoder.
//
// Two levels of status words.  A tile's is its own block_info, read and written as one 64-bit word
// {u32 offset; u16 byte_num; u16 state}: a launch before this one marks every tile KVC_BI_NOT_READY, a wave that
// knows its size writes {0, byte_num, KVC_BI_SIZE}, and once it knows its offset the final {offset, byte_num, 0}
// (the reference's layout, state = padding = 0).  Runs of 56 consecutive tiles form a group with a word
// {u32 bytes; u32 state} in the call's scratch slot: the wave of a group's last tile adds up the group
// (KVC_BI_SIZE) and, once it knows what lies in front of the group, publishes the bytes up to the group's end
// (state 0).  So a wave reads the sizes of the tiles before it in its own group (one 64-lane look), then walks the
// group words backwards, 64 per look, adding sizes until a group with a known end stops the walk; tiles in flight
// span a few dozen groups, so that is one or two looks.  Words that are not ready are polled again.
//
// Progress.  Two rules make every wait end: (1) a workgroup takes its tiles from a ticket counter when it starts
// (not from its index in the launch, whose order of execution HIP does not promise), so every tile before a wave's
// own belongs to a workgroup that has started; (2) a wave waits for nothing until the sizes of ALL its tiles are
// published, and a group's size only needs the sizes of its own tiles.  So whatever a wave waits for is published
// by waves that are running and wait for nothing before they publish.  (Placing a run's first tile before its
// second was counted breaks rule 2 and turns the launch into one chain from wave to wave: 18 ms instead of 0.2.)
// A wave that has found a word not ready more than max_polls times gives up all the same, flags the call
// (KVC_ENC_ERR_ORDER) and publishes what it has, so that every wave ends; kvc_encode_finish_kernel then encodes the
// whole call again the slow, safe way (two passes inside one workgroup), so a give-up costs time, not the result.
constexpr uint32_t KVC_BI_SIZE = 1u, KVC_BI_NOT_READY = 0xffffu;
constexpr uint32_t KVC_ENC_ERR_ORDER = 16u;         // a tile waited too long for the tiles before it
constexpr uint32_t KVC_NO_CODE_LEN = 0x4000u;       // length of a symbol without a code: shows in any sum of lengths
// The scratch slot of a one-pass call, in 32-bit words.  Tens of thousands of waves read the first tile's offset and
// thousands of workgroups report maxima: on one cache line those accesses queue up behind each other (measured:
// 0.5 ms of a 1.1 ms launch), so the offset gets a line that nothing is written to while the kernel runs, and the
// maxima go to one of 32 lines picked by the workgroup number (kvc_encode_finish_kernel joins them afterwards).
// The ticket counter shares the line of the call's status words, which nobody touches before the last tile is placed.
constexpr int KVC_ONCE_POLLS_WORD = 6;               // status word: most looks of one wave that found a word not ready
constexpr int KVC_ONCE_TICKET_WORD = 16;             // workgroups started so far
constexpr int KVC_ONCE_BASE_WORD = 32;               // copy of status[KVC_ENC_ST_BASE]
constexpr int KVC_ONCE_PART_WORD = 64, KVC_ONCE_PART_LINES = 32, KVC_ONCE_PART_STRIDE = 32;   // {error bits, largest tile, longest stream, polls}
constexpr int KVC_ONCE_GROUP_WORD = KVC_ONCE_PART_WORD + KVC_ONCE_PART_LINES * KVC_ONCE_PART_STRIDE;
constexpr int KVC_ONCE_MAX_GROUPS = (int)((KVC_WS_SLOT_BYTES - KVC_ONCE_GROUP_WORD * 4) / 8);
// Tiles per group: seven workgroups of a run-of-two launch, not eight.  Workgroups go to the chip's eight dies in turn,
// and the wave of a group's last tile waits for its whole group before it publishes the group's size: with groups of
// eight workgroups all of those waves sit on one die, that die falls behind, and the seven others wait for it at every
// group (measured: 10 us per wave there, 3 us on the die with the last tiles).
constexpr int KVC_ONCE_GROUP_TILES = 56;
static_assert(KVC_ONCE_GROUP_TILES <= KVC_WAVE && KVC_ONCE_GROUP_TILES % 2 == 0, "one look of 64 lanes covers a group; a run of two stays inside one");
__device__ __forceinline__ int64_t kvc_once_group(int64_t tile) { return (int64_t)((uint32_t)tile / (uint32_t)KVC_ONCE_GROUP_TILES); }
__device__ __forceinline__ bool kvc_once_closes(const KvcEncodeArgs &a, int64_t tile)
{
    return (uint32_t)tile % (uint32_t)KVC_ONCE_GROUP_TILES == (uint32_t)KVC_ONCE_GROUP_TILES - 1u || tile == a.tiles - 1;
}

__device__ __forceinline__ uint64_t kvc_bi_word(uint32_t offset, uint32_t byte_num, uint32_t state)
{
    return (uint64_t)offset | ((uint64_t)(byte_num & 0xffffu) << 32) | ((uint64_t)state << 48);
}
__device__ __forceinline__ uint64_t kvc_group_word(uint32_t bytes, uint32_t state) { return (uint64_t)bytes | ((uint64_t)state << 32); }
__device__ __forceinline__ uint64_t *kvc_group_words(const KvcEncodeArgs &a)
{
    return reinterpret_cast<uint64_t *>(a.status + KVC_ONCE_GROUP_WORD);
}
__device__ __forceinline__ uint64_t kvc_status_load(const uint64_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void kvc_status_store(uint64_t *p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ uint32_t kvc_wave_sum_u32(uint32_t v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += (uint32_t)__shfl_xor((int)v, o, 64);
    return v;
}

__global__ void __launch_bounds__(KVC_WG) kvc_encode_mark_kernel(KvcEncodeArgs a)
{
    const int64_t tile = (int64_t)blockIdx.x * KVC_WG + threadIdx.x;
    if (tile < a.tiles) reinterpret_cast<uint64_t *>(a.block_infos)[tile] = kvc_bi_word(0u, 0u, KVC_BI_NOT_READY);
    if (tile < (a.tiles + KVC_ONCE_GROUP_TILES - 1) / KVC_ONCE_GROUP_TILES) kvc_group_words(a)[tile] = kvc_group_word(0u, KVC_BI_NOT_READY);
    if (blockIdx.x == 0) {
        for (int i = threadIdx.x; i < KVC_ONCE_PART_LINES * KVC_ONCE_PART_STRIDE; i += KVC_WG) a.status[KVC_ONCE_PART_WORD + i] = 0u;
        if (threadIdx.x == 0) {
            a.status[KVC_ONCE_BASE_WORD] = a.status[KVC_ENC_ST_BASE];
            a.status[KVC_ONCE_TICKET_WORD] = 0u;
        }
    }
}

// What a wave asks for as soon as it has published its size, and looks at only after it has packed its payload: the
// words of the tiles before it in its group and of the 64 groups before its own.  The two round trips then run
// while the wave works, and by the time it looks the words are usually final.
struct KvcFirstLooks {
    uint64_t tile_word, group_word;
};

__device__ __forceinline__ KvcFirstLooks kvc_look_back_ask(const KvcEncodeArgs &a, int64_t tile, int lane)
{
    const uint64_t *bi64 = reinterpret_cast<const uint64_t *>(a.block_infos);
    const int64_t group = kvc_once_group(tile);
    const int r = (int)(tile - group * KVC_ONCE_GROUP_TILES);
    KvcFirstLooks f;
    f.tile_word = lane < r ? kvc_status_load(bi64 + group * KVC_ONCE_GROUP_TILES + lane) : 0ull;
    f.group_word = group - 1 - lane >= 0 ? kvc_status_load(kvc_group_words(a) + group - 1 - lane) : kvc_group_word(0u, 0u);
    return f;
}

// First half of the look-back: the payload bytes of the tiles before `tile` in its own group; the wave of a group's last
// tile then publishes the group's size.  *polls counts the looks that found a word not ready (wave-uniform).
__device__ __forceinline__ uint32_t kvc_look_back_in_group(const KvcEncodeArgs &a, int64_t tile, uint32_t bn, int lane, uint64_t first_look,
                                                           int *polls)
{
    const uint64_t *bi64 = reinterpret_cast<const uint64_t *>(a.block_infos);
    const int64_t group = kvc_once_group(tile);
    const int r = (int)(tile - group * KVC_ONCE_GROUP_TILES);
    uint32_t in_group = 0;
    uint64_t w = first_look;
    while (r > 0) {
        if (!__any((uint32_t)(w >> 48) == KVC_BI_NOT_READY)) {
            in_group = kvc_wave_sum_u32(lane < r ? (uint32_t)(w >> 32) & 0xffffu : 0u);
            break;
        }
        if (++*polls > a.max_polls) break;
        __builtin_amdgcn_s_sleep(2);
        w = lane < r ? kvc_status_load(bi64 + group * KVC_ONCE_GROUP_TILES + lane) : 0ull;
    }
    if (kvc_once_closes(a, tile) && lane == 0)             // this wave speaks for its group
        kvc_status_store(kvc_group_words(a) + group, kvc_group_word(in_group + bn, KVC_BI_SIZE));
    return in_group;
}

// Second half: the payload bytes of the groups before the tile's own; the wave of a group's last tile then publishes
// the bytes up to the end of its group.
__device__ __forceinline__ uint32_t kvc_look_back_groups(const KvcEncodeArgs &a, int64_t tile, uint32_t in_group_and_own, int lane,
                                                         uint64_t first_look, int *polls)
{
    uint64_t *groups = kvc_group_words(a);
    const int64_t group = kvc_once_group(tile);
    uint32_t before = 0;
    int64_t j = group - 1;                                 // nearest group not yet accounted for
    uint64_t w = first_look;                               // taken at j = group - 1
    while (j >= 0 && *polls <= a.max_polls) {
        const uint32_t state = (uint32_t)(w >> 32), bytes = (uint32_t)w;
        const uint64_t not_ready = __ballot(state == KVC_BI_NOT_READY), known = __ballot(state == 0u);
        const int first_nr = not_ready ? __builtin_ctzll(not_ready) : 64, first_kn = known ? __builtin_ctzll(known) : 64;
        const int stop = first_kn < first_nr ? first_kn + 1 : first_nr;     // lanes below it count: sizes, then maybe an end
        before += kvc_wave_sum_u32(lane < stop ? bytes : 0u);
        if (first_kn < first_nr) break;                    // a group whose end is known closes the sum
        j -= stop;
        if (first_nr < 64) {
            ++*polls;
            __builtin_amdgcn_s_sleep(2);
        }
        const int64_t idx = j - lane;
        w = idx >= 0 ? kvc_status_load(groups + idx) : kvc_group_word(0u, 0u);   // in front of the first group: nothing, and known
    }
    if (kvc_once_closes(a, tile) && lane == 0)
        kvc_status_store(groups + group, kvc_group_word(before + in_group_and_own, 0u));
    return before;
}

// A wave's (or the workgroup's) copy of the encode table for the one-pass kernel: as kvc_load_code_table, but an
// entry without a usable code gets the length KVC_NO_CODE_LEN.
__device__ __forceinline__ void kvc_load_code_table_marked(const KvcEncodeArgs &a, int64_t tile, uint2 *s_table, uint32_t *s_short, int lane)
{
    const uint2 *t = reinterpret_cast<const uint2 *>(kvc_table_of_row(a, tile / a.cols));
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int i = lane + KVC_WAVE * k;
        uint2 e = i < a.table_entries ? t[i] : make_uint2(0u, 0u);
        if (e.y == 0u || e.y > 32u) e = make_uint2(0u, KVC_NO_CODE_LEN);
        else if (e.y < 32u) e.x &= (1u << e.y) - 1u;      // nothing above the code's own bits
        s_table[i] = e;
        if (e.y > 8u && e.y != KVC_NO_CODE_LEN) atomicAnd(s_short, 0u);
    }
}

// LDS of one wave of the one-pass kernel: for V from fp16 the tokens' constants, then one area that holds the payload
// images from its start upwards and the staging area of the tile front end at its top.  A payload of any size (at
// most KVC_MAX_TILE_BYTES) leaves the staging area free, so a run's first tile can always wait in LDS while the second
// is staged and counted; the second tile's image goes behind the first one's when both fit (it may then run into the
// staging area, which is free by then), and otherwise the first tile is placed and written out before the second is
// packed -- with both sizes published long before, so that nobody waits for this wave in the meantime.
constexpr int KVC_ONCE_WAVE_BYTES = 12560;               // three workgroups of four waves per compute unit (160 KB)
constexpr int kvc_once_par_bytes(int front) { return front == 2 ? 4 * KVC_V_TOKENS * 4 : 0; }
constexpr int kvc_once_stage_bytes(int front) { return front == 1 ? KVC_STAGE_K_BYTES : front == 2 ? KVC_STAGE_VF16_BYTES : KVC_STAGE_VSYM_BYTES; }
constexpr int kvc_once_area_bytes(int front) { return KVC_ONCE_WAVE_BYTES - kvc_once_par_bytes(front); }
static_assert(KVC_STAGE_VSYM_BYTES >= KVC_STAGE_K_BYTES, "symbols in: the staging area serves K and V tiles");
static_assert(kvc_once_area_bytes(0) - kvc_once_stage_bytes(0) >= KVC_IMAGE_WORDS * 4 &&
              kvc_once_area_bytes(1) - kvc_once_stage_bytes(1) >= KVC_IMAGE_WORDS * 4 &&
              kvc_once_area_bytes(2) - kvc_once_stage_bytes(2) >= KVC_IMAGE_WORDS * 4, "the largest payload must leave the staging area free");
__device__ __forceinline__ uint32_t kvc_once_image_words(uint32_t bn) { return (bn + 3u) / 4u + 1u; }

// A tile whose payload is packed but not yet placed; the words its look-back reads were asked for when its size was
// published.
struct KvcOncePending {
    int64_t tile;                                          // -1: nothing pending
    uint32_t bn, in_group;
    bool in_group_known, packs;
    KvcFirstLooks looks;
};

// Find where a tile whose size has been published goes (by looking back, or -- `follows` -- right behind the tile
// before it, which this wave has just placed at follows_off), publish its block_info and write its payload from the LDS
// image (which starts on a word; the payload lands p.head bytes into an aligned word).  Returns error bits; *off_out
// receives the tile's global offset.
__device__ __forceinline__ uint32_t kvc_once_place(const KvcEncodeArgs &a, const KvcOncePending &pd, const uint32_t *image, uint32_t base,
                                                   int lane, int *polls, uint32_t *off_out, bool follows = false, uint32_t follows_off = 0)
{
    const int64_t tile = pd.tile;
    const uint32_t bn = pd.bn;
    uint32_t off;
    if (follows) {
        off = follows_off;
        if (kvc_once_closes(a, tile) && lane == 0)         // this wave speaks for its group: the group's end
            kvc_status_store(kvc_group_words(a) + kvc_once_group(tile), kvc_group_word(off + bn - base, 0u));
    } else {
        uint32_t in_group = pd.in_group;
        if (!pd.in_group_known) in_group = kvc_look_back_in_group(a, tile, bn, lane, pd.looks.tile_word, polls);
        off = base + in_group + kvc_look_back_groups(a, tile, in_group + bn, lane, pd.looks.group_word, polls);
    }
    *off_out = off;
    uint32_t err = 0;
    const bool gave_up = *polls > a.max_polls;
    if (lane == 0) kvc_status_store(reinterpret_cast<uint64_t *>(a.block_infos) + tile, kvc_bi_word(off, bn, 0u));
    if (gave_up) err |= KVC_ENC_ERR_ORDER;
    KvcEmitPlace p;
    p.off = off - a.base_global_offset;
    p.bn = bn;
    p.ok = !gave_up && pd.packs && (int64_t)p.off + bn <= a.encoded_cap;
    p.head = p.ok ? (uint32_t)((reinterpret_cast<uintptr_t>(a.encoded) + p.off) & 3u) : 0u;
    if (tile == a.tiles - 1 && lane == 0) {                // the call's totals, by the wave of the last tile
        const uint32_t total = off + bn - base;
        a.status[0] = total;
        if ((int64_t)(base - a.base_global_offset) + total > a.encoded_cap) err |= KVC_ENC_ERR_CAPACITY;
        if (a.idx_offset) {
            a.idx_offset[0] = (uint32_t)a.tiles;
            a.idx_offset[1] = total;
        }
    }
    if (p.ok) kvc_write_image_shifted(a, p, lane, image);
    return err;
}

// FRONT 0: uint8 symbols in; 1: fp16 K tile (quantized here); 2: fp16 V tile.
// A wave works through `run` (one or two) consecutive tiles.  For each it counts (symbols -> codes and lengths,
// thread_infos), publishes the size, asks for the words its look-back will read and packs the payload into LDS as an
// image that starts on a word (where the payload goes is not needed for that).  The first tile of a run of two stays in
// LDS until the second is counted and packed too; then one look-back finds the first tile's place, the second
// follows right behind it, and both are written out.  So a tile is placed a whole tile's work after its size was
// published, when the tiles before it have published theirs: with the look-back right behind the count, a tile waits
// 10 us on average for the slowest of the thousands of tiles in flight before it (measured), as long as the rest of
// its work takes.
// Dynamic LDS: the encode table (one for the workgroup, or one per wave when tile rows have codebooks of their own:
// then run = 1), then KVC_ONCE_WAVE_BYTES per wave.
template <int FRONT>
__global__ void __launch_bounds__(KVC_WG, 3) kvc_encode_once_kernel(KvcStoreArgs a, int run)
{
    extern __shared__ __align__(16) uint8_t s_dyn[];
    __shared__ uint32_t s_short[KVC_WAVES_PER_WG], s_err, s_max_tile, s_longest, s_polls, s_ticket;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool own_table = a.e.rows_per_codebook != 0;
    uint2 *s_table = reinterpret_cast<uint2 *>(s_dyn) + (own_table ? wave * 256 : 0);
    uint8_t *s_wave = s_dyn + (own_table ? KVC_WAVES_PER_WG : 1) * 256 * sizeof(uint2) + wave * KVC_ONCE_WAVE_BYTES;
    constexpr int PAR_BYTES = kvc_once_par_bytes(FRONT), AREA_BYTES = kvc_once_area_bytes(FRONT);
    uint32_t *s_par = reinterpret_cast<uint32_t *>(s_wave);
    uint32_t *area = reinterpret_cast<uint32_t *>(s_wave + PAR_BYTES);
    uint8_t *s_stage = s_wave + PAR_BYTES + AREA_BYTES - kvc_once_stage_bytes(FRONT);
    uint32_t *my_short = &s_short[own_table ? wave : 0];
    // the workgroup's ticket: which tiles it takes (the table of a call with one codebook is fetched meanwhile)
    uint32_t ticket = 0;
    if (tid == 0) ticket = atomicAdd(&a.e.status[KVC_ONCE_TICKET_WORD], 1u);
    if (lane == 0) s_short[wave] = 1u;
    if (!own_table && wave == 0) kvc_load_code_table_marked(a.e, 0, s_table, my_short, lane);
    if (tid == 0) { s_err = 0; s_max_tile = 0; s_longest = 0; s_polls = 0; s_ticket = ticket; }
    __syncthreads();
    const int64_t tile0 = ((int64_t)s_ticket * KVC_WAVES_PER_WG + wave) * run;
    if (own_table) {
        if (tile0 < a.e.tiles) kvc_load_code_table_marked(a.e, tile0, s_table, my_short, lane);
        __syncthreads();
    }
    const bool short_codes = *my_short != 0u;              // wave-uniform
    uint64_t *bi64 = reinterpret_cast<uint64_t *>(a.e.block_infos);
    const uint32_t base = a.e.status[KVC_ONCE_BASE_WORD];
    uint32_t err = 0, max_tile = 0, longest = 0, next_off = 0;
    int polls = 0;
    bool first_placed = false;
    KvcOncePending pd;
    pd.tile = -1;
    uint32_t raw[KVC_WAVE];                                // a tile as loaded from fp16: two channels of 64 tokens per lane
#pragma unroll 1
    for (int it = 0; it < run; it++) {
        const int64_t tile = tile0 + it;
        if (tile >= a.e.tiles) break;
        // (the lane number made opaque: what the front ends derive from it -- some dozens of LDS and global addresses --
        // is then worked out where it is used instead of being kept in registers across the whole loop body)
        int lane = tid & 63;
        asm volatile("" : "+v"(lane));
        // (and the arguments are read again per tile rather than kept in scalar registers through everything; so is the
        // word count of a vector, or the 32 comparisons "word j belongs to the vector" would be worked out once for the
        // whole kernel and kept as 32 lane masks, most of them spilled)
        const KvcStoreArgs &a = kvc_kernarg_again<KvcStoreArgs>();
        int nd = a.e.vec_len >> 2;
        asm volatile("" : "+s"(nd));
        uint32_t v[32];
        if constexpr (FRONT == 1) {
            // the loads of the run's second tile are on their way while the first is counted and packed
            if (it == 0) kvc_front_k_load(a, tile, lane, raw);
            kvc_front_k_once(a, tile, lane, s_stage, raw, v);
            if (it + 1 < run && tile + 1 < a.e.tiles) kvc_front_k_load(a, tile + 1, lane, raw);
        } else if constexpr (FRONT == 2) {
            if (it == 0) kvc_front_v_load(a, tile, lane, raw);
            kvc_front_v(a, tile, lane, s_stage, s_par, raw, v);
            if (it + 1 < run && tile + 1 < a.e.tiles) kvc_front_v_load(a, tile + 1, lane, raw);
        } else {
            if (a.e.is_k) kvc_load_vector_k_tile(a.e, tile, lane, s_stage, v);
            else kvc_load_vector_v_tile(a.e, tile, lane, s_stage, v);       // (the launcher requires 4-byte aligned symbols and rows)
        }
        // (every lane holds its vector and the staging area is free: the front ends finish with a hand-over)
        uint32_t bits = 0;
        uint32_t gl[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u}; // short codes: the four group lengths of registers 4 i .. 4 i + 3
        if (short_codes) {
#pragma unroll
            for (int j = 0; j < 32; j++) {
                if (j < nd) {
                    const uint2 e0 = s_table[v[j] & 0xffu], e1 = s_table[(v[j] >> 8) & 0xffu];
                    const uint2 e2 = s_table[(v[j] >> 16) & 0xffu], e3 = s_table[v[j] >> 24];
                    const uint32_t len = e0.y + e1.y + e2.y + e3.y;
                    // (the marked length of a symbol without a code shifts by nothing)
                    v[j] = ((((e0.x << (e1.y & 31u)) | e1.x) << (e2.y & 31u) | e2.x) << (e3.y & 31u)) | e3.x;
                    bits += len;
                    gl[j >> 2] |= (len & 0xffu) << (8 * (j & 3));
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 32; j++) {
                if (j < nd) {
#pragma unroll
                    for (int k = 0; k < 4; k++) bits += s_table[(v[j] >> (8 * k)) & 0xffu].y;
                }
            }
        }
        const bool bad = bits >= KVC_NO_CODE_LEN;          // a symbol without a code: the lane emits nothing
        if (bad) bits = 0;
        const uint32_t bytes = (bits + 7u) >> 3;
        const uint32_t end = kvc_wave_inclusive_scan(bytes, lane);
        a.e.thread_infos[tile * KVC_WAVE + lane] = (uint16_t)((end << 3) + (bytes << 3) - bits);
        const uint32_t start = end - bytes;
        const uint32_t tile_bytes = (uint32_t)__builtin_amdgcn_readlane((int)end, KVC_WAVE - 1);
        const uint32_t bn = tile_bytes > 0xffffu ? 0xffffu : tile_bytes;
        if (__any(bad)) err |= KVC_ENC_ERR_NO_CODE;
        if (tile_bytes > (uint32_t)KVC_MAX_TILE_BYTES) err |= KVC_ENC_ERR_TILE_TOO_BIG;
        const uint32_t lg = kvc_wave_max_dpp(bytes);
        longest = lg > longest ? lg : longest;
        max_tile = bn > max_tile ? bn : max_tile;
        if (lane == 0) kvc_status_store(bi64 + tile, kvc_bi_word(0u, bn, KVC_BI_SIZE));
        KvcOncePending cur;
        cur.tile = tile;
        cur.bn = bn;
        // the wave that speaks for a group must not sit on the group's size (the groups after it wait for that word,
        // and so would, one after the other, the waves that speak for them): it adds up its group at once
        cur.in_group_known = kvc_once_closes(a.e, tile);
        cur.in_group = 0;
        cur.looks.tile_word = cur.looks.group_word = 0ull;
        if (pd.tile < 0 || cur.in_group_known) cur.looks = kvc_look_back_ask(a.e, tile, lane);    // (a tile that follows a kept one looks at nothing)
        if (cur.in_group_known) cur.in_group = kvc_look_back_in_group(a.e, tile, bn, lane, cur.looks.tile_word, &polls);
        cur.packs = bn <= (uint32_t)KVC_MAX_TILE_BYTES;
        // where this tile's image goes: behind the kept one's, or -- the two do not fit the area together (more than six
        // bits per symbol on average) -- to the start of the area once the kept tile has been placed and written out.
        // The sizes of both tiles are published by now: this wave's wait holds nobody up.
        const uint32_t my_words = kvc_once_image_words(bn);
        uint32_t *image = area;
        if (pd.tile >= 0) {
            const uint32_t kept_words = pd.packs ? kvc_once_image_words(pd.bn) : 0u;
            if (cur.packs && (kept_words + my_words) * 4u > (uint32_t)AREA_BYTES) {
                uint32_t off = 0;
                err |= kvc_once_place(a.e, pd, area, base, lane, &polls, &off);
                next_off = off + pd.bn;
                first_placed = true;
                pd.tile = -1;
                kvc_wave_lds_sync();                       // the kept image is read: the area is free
            } else {
                image = area + kept_words;
            }
        }
        if (cur.packs) {
            for (uint32_t i = lane; i < my_words; i += KVC_WAVE) image[i] = 0;
            kvc_wave_lds_sync();
            if (short_codes) {
                const uint32_t bitpos = start * 8u;
                uint32_t w = bitpos >> 5, nacc = bitpos & 31u;
                uint64_t acc = 0;
                if (!bad) {
#pragma unroll
                    for (int j = 0; j < 32; j++) {
                        if (j < nd) {
                            const uint32_t len = (gl[j >> 2] >> (8 * (j & 3))) & 0xffu;
                            acc = (acc << len) | v[j];
                            nacc += len;
                            if (nacc >= 32u) {
                                nacc -= 32u;
                                if (w < my_words) atomicOr(&image[w], kvc_bswap((uint32_t)(acc >> nacc)));
                                w++;
                            }
                        }
                    }
                    if (nacc > 0 && w < my_words) atomicOr(&image[w], kvc_bswap((uint32_t)(acc << (32u - nacc))));
                }
            } else if (!bad) {
                kvc_pack_vector(a.e, start, v, s_table, image, 0u, false, my_words);
            }
            kvc_wave_lds_sync();
        }
        if (it + 1 < run && tile + 1 < a.e.tiles) {
            pd = cur;                                      // placed together with the next tile
            continue;
        }
        uint32_t off = 0;
        if (pd.tile >= 0) {                                // the kept tile, whose words have had this tile's work to arrive
            err |= kvc_once_place(a.e, pd, area, base, lane, &polls, &off);
            err |= kvc_once_place(a.e, cur, image, base, lane, &polls, &off, true, off + pd.bn);
            pd.tile = -1;
        } else if (first_placed) {                         // the kept tile went out before this one was packed
            err |= kvc_once_place(a.e, cur, image, base, lane, &polls, &off, true, next_off);
        } else {                                           // a run of one
            err |= kvc_once_place(a.e, cur, image, base, lane, &polls, &off);
        }
    }
    if (lane == 0 && tile0 < a.e.tiles) {
        if (err) atomicOr(&s_err, err);
        atomicMax(&s_max_tile, max_tile);
        atomicMax(&s_longest, longest);
        atomicMax(&s_polls, (uint32_t)polls);
    }
    __syncthreads();
    if (tid == 0) {                                        // to one of the slot's lines, picked by the ticket
        uint32_t *part = a.e.status + KVC_ONCE_PART_WORD + (s_ticket % KVC_ONCE_PART_LINES) * KVC_ONCE_PART_STRIDE;
        if (s_err) atomicOr(&part[0], s_err);
        atomicMax(&part[1], s_max_tile);
        atomicMax(&part[2], s_longest);
        atomicMax(&part[3], s_polls);
    }
}

// After the one-pass kernel, one workgroup: joins what the workgroups reported on their 32 lines into the call's status
// words.  If a wave gave up on its look-back (KVC_ENC_ERR_ORDER: the payload and the block_infos are then incomplete)
// this workgroup encodes the whole call again in two passes of its own -- count every tile, add up the offsets, emit
// every tile: nothing in it waits for another workgroup, so it always ends, and since the inputs are untouched the
// outputs are the ones the call was to produce.  Slow (four waves for all tiles), and next to never needed: the
// look-back's progress does not depend on the order in which the hardware starts workgroups.
template <int FRONT>
__global__ void __launch_bounds__(KVC_WG) kvc_encode_finish_kernel(KvcStoreArgs a)
{
    __shared__ uint2 s_table[KVC_WAVES_PER_WG][256];
    __shared__ uint8_t s_len[KVC_WAVES_PER_WG][256];
    __shared__ __align__(16) uint8_t s_sym[KVC_WAVES_PER_WG][KVC_SYM_TILE_BYTES];   // staging area first, then the payload image
    __shared__ __align__(16) uint32_t s_par[FRONT == 2 ? KVC_WAVES_PER_WG : 1][FRONT == 2 ? 4 * KVC_V_TOKENS : 4];
    __shared__ uint32_t s_short[KVC_WAVES_PER_WG], s_err, s_longest, s_again;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (wave == 0) {
        uint32_t err = 0, tile = 0, stream = 0, polls = 0;
        if (lane < KVC_ONCE_PART_LINES) {
            const uint32_t *p = a.e.status + KVC_ONCE_PART_WORD + lane * KVC_ONCE_PART_STRIDE;
            err = p[0];
            tile = p[1];
            stream = p[2];
            polls = p[3];
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            err |= (uint32_t)__shfl_xor((int)err, o, 64);
            const uint32_t t = (uint32_t)__shfl_xor((int)tile, o, 64), st = (uint32_t)__shfl_xor((int)stream, o, 64);
            const uint32_t po = (uint32_t)__shfl_xor((int)polls, o, 64);
            tile = t > tile ? t : tile;
            stream = st > stream ? st : stream;
            polls = po > polls ? po : polls;
        }
        if (a.e.force_order) err |= KVC_ENC_ERR_ORDER;
        if (lane == 0) {
            a.e.status[KVC_ONCE_POLLS_WORD] = polls;
            s_again = err & KVC_ENC_ERR_ORDER;
            if (!(err & KVC_ENC_ERR_ORDER)) {
                a.e.status[1] |= err;
                a.e.status[2] = tile;
                a.e.status[3] = stream;
            }
            s_err = 0;
            s_longest = 0;
        }
    }
    __syncthreads();
    if (!s_again) return;
    // ---- the whole call again, two passes inside this workgroup ----
    const int64_t tiles = a.e.tiles;
    for (int64_t tile = wave; tile < tiles; tile += KVC_WAVES_PER_WG) {      // count: thread_infos, byte_nums, group parameters
        kvc_load_len_table(a.e, tile, s_len[wave], lane);
        kvc_wave_lds_sync();
        uint32_t v[32];
        if constexpr (FRONT == 1) {
            uint32_t raw[KVC_WAVE];
            kvc_front_k_load(a, tile, lane, raw);
            kvc_front_k_once(a, tile, lane, s_sym[wave], raw, v);
        } else if constexpr (FRONT == 2) {
            uint32_t raw[KVC_WAVE];
            kvc_front_v_load(a, tile, lane, raw);
            kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], raw, v);
        } else {
            kvc_load_vector(a.e, tile, lane, v);
        }
        const uint32_t longest = kvc_count_tile(a.e, tile, lane, v, s_len[wave], &s_err);
        if (lane == 0) atomicMax(&s_longest, longest);
        kvc_wave_lds_sync();
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (wave == 0) {                                                         // offsets, in tile order
        uint32_t *bi = reinterpret_cast<uint32_t *>(a.e.block_infos);
        const uint32_t base = a.e.status[KVC_ENC_ST_BASE];
        uint32_t at = base, largest = 0;
        for (int64_t t0 = 0; t0 < tiles; t0 += KVC_WAVE) {
            const int64_t tile = t0 + lane;
            const uint32_t bn = tile < tiles ? bi[2 * tile + 1] & 0xffffu : 0u;
            const uint32_t incl = kvc_wave_inclusive_scan(bn, lane);
            if (tile < tiles) bi[2 * tile] = at + incl - bn;
            at += (uint32_t)__builtin_amdgcn_readlane((int)incl, KVC_WAVE - 1);
            const uint32_t m = kvc_wave_max_dpp(bn);
            largest = m > largest ? m : largest;
        }
        if (lane == 0) {
            const uint32_t total = at - base;
            a.e.status[0] = total;
            a.e.status[2] = largest;
            if ((int64_t)(base - a.e.base_global_offset) + total > a.e.encoded_cap) atomicOr(&s_err, KVC_ENC_ERR_CAPACITY);
            if (a.e.idx_offset) {
                a.e.idx_offset[0] = (uint32_t)tiles;
                a.e.idx_offset[1] = total;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    for (int64_t tile = wave; tile < tiles; tile += KVC_WAVES_PER_WG) {      // emit
        if (lane == 0) s_short[wave] = 1u;
        kvc_wave_lds_sync();
        kvc_load_code_table(a.e, tile, s_table[wave], &s_short[wave], lane);
        kvc_wave_lds_sync();
        const KvcEmitPlace p = kvc_emit_place(a.e, tile, true);
        if (!p.ok) continue;                                                 // flagged by the count pass or the offsets
        uint32_t *image = reinterpret_cast<uint32_t *>(s_sym[wave]);
        uint32_t v[32];
        if constexpr (FRONT == 1) {
            kvc_front_k(a, tile, lane, s_sym[wave], v);
        } else if constexpr (FRONT == 2) {
            uint32_t raw[KVC_WAVE];
            kvc_front_v_load(a, tile, lane, raw);
            kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], raw, v);
        } else {
            kvc_load_vector(a.e, tile, lane, v);
        }
        kvc_wave_lds_sync();
        const uint32_t image_words = (p.head + p.bn + 3u) / 4u + 1u;
        for (uint32_t i = lane; i < image_words && i < (uint32_t)KVC_IMAGE_WORDS; i += KVC_WAVE) image[i] = 0;
        kvc_wave_lds_sync();
        kvc_pack_vector(a.e, kvc_stream_start(a.e, tile, lane), v, s_table[wave], image, p.head, s_short[wave] != 0u);
        kvc_wave_lds_sync();
        kvc_write_image(a.e, p, lane, image);
        kvc_wave_lds_sync();
    }
    __syncthreads();
    if (tid == 0) {
        a.e.status[1] = (a.e.status[1] & KVC_ENC_ERR_CODEBOOK) | s_err;
        a.e.status[3] = s_longest;
    }
}

// What the fused path adds to an encode call: the fp16 source and how to quantize it.
struct KvcStoreSource {
    const void *x_f16;
    int64_t B, H;
    int mask;
    float eb;
    int8_t *min_i8;
    void *scale_f16;
};

// Everything an encode call is made of; the classic entry points fill in what they have and leave the rest zero.
struct KvcEncodeCall {
    int is_k;
    const uint8_t *d_sym;
    int64_t tokens, stride, head_dim;
    const uint8_t *d_tables;
    int64_t table_bytes, table_stride, rows_per_codebook;
    const int32_t *d_meta;
    uint8_t *d_block_infos, *d_thread_infos, *d_idx_offset, *d_encoded;
    int64_t encoded_cap;
    uint32_t base_global_offset;
    uint32_t *d_stream_bytes, *d_result;
    const KvcStoreSource *src;
};

static int kvc_encode_errors(uint32_t bits, uint32_t total, int64_t encoded_cap)
{
    if (bits & KVC_ENC_ERR_CODEBOOK) return kvc_fail(-3, "a codebook of this call was not built (fewer than two symbols, or not representable)");
    if (bits & KVC_ENC_ERR_NO_CODE) return kvc_fail(-3, "a symbol has no code in the encode table");
    if (bits & KVC_ENC_ERR_TILE_TOO_BIG)
        return kvc_fail(-3, "a tile encodes to more than %d bytes, which thread_info (u16) cannot address", KVC_MAX_TILE_BYTES);
    if (bits & KVC_ENC_ERR_CAPACITY)
        return kvc_fail(-3, "payload (%u bytes) does not fit the encoded_data buffer (%lld bytes)", total, (long long)encoded_cap);
    if (bits & KVC_ENC_ERR_ORDER) return kvc_fail(-3, "one-pass encoder: a tile waited too long for the tiles before it");
    return 0;
}

// Queue the launches of one encode call (init, count, per-1024-tile sums, offsets, emit, publish); waits for nothing.
// *slot receives the call's status words on the device.
static int kvc_encode_launch(const KvcEncodeCall &c, void **slot_out, hipStream_t stream)
{
    int64_t sizes[4];
    if (int rc = kvc_calculate_buffer_size(c.tokens, c.stride, c.is_k, 0, c.head_dim, sizes)) return rc;
    KVC_REQUIRE(c.tokens > 0, "nothing to encode");
    KVC_REQUIRE(c.head_dim % 8 == 0, "head_dim must be a multiple of 8");
    KVC_REQUIRE(c.table_bytes > 0 && c.table_bytes % 8 == 0 && c.table_bytes <= 256 * 8,
                "encode table must hold 1..256 entries of 8 bytes");
    KVC_REQUIRE(((uintptr_t)c.d_tables & 7) == 0 && ((uintptr_t)c.d_block_infos & 3) == 0 &&
                ((uintptr_t)c.d_thread_infos & 1) == 0 && ((uintptr_t)c.d_idx_offset & 3) == 0 && ((uintptr_t)c.d_sym & 3) == 0 &&
                ((uintptr_t)c.d_stream_bytes & 3) == 0 && ((uintptr_t)c.d_result & 3) == 0,
                "encode buffers are misaligned");
    KVC_REQUIRE(c.src != nullptr || c.d_sym != nullptr, "symbol pointer is NULL");
    KVC_REQUIRE(c.stride % 4 == 0, "stride must be a multiple of 4");
    KVC_REQUIRE(c.rows_per_codebook >= 0 && (c.rows_per_codebook == 0 || (c.table_stride >= c.table_bytes && c.table_stride % 8 == 0)),
                "tables of several codebooks must be a multiple of 8 bytes apart and not overlap");
    void *slot;
    if (int rc = kvc_workspace_slot(&slot, (void *)stream)) return rc;
    KvcEncodeArgs a;
    a.sym = c.d_sym;
    a.stride = c.stride;
    a.is_k = c.is_k;
    a.vec_len = c.is_k ? (int)c.head_dim : KVC_V_TOKENS;
    a.cols = (int)(c.is_k ? c.stride / c.head_dim : c.stride / KVC_V_VEC_PER_BLK);
    a.tiles = sizes[0] / 8;
    a.table = c.d_tables;
    a.table_entries = (int)(c.table_bytes / 8);
    a.table_stride = c.table_stride;
    a.rows_per_codebook = (int)c.rows_per_codebook;
    a.codebook_meta = c.d_meta;
    const int64_t rows = a.tiles / a.cols;
    a.n_codebooks = c.rows_per_codebook ? (int)((rows + c.rows_per_codebook - 1) / c.rows_per_codebook) : 1;
    a.block_infos = c.d_block_infos;
    a.thread_infos = reinterpret_cast<uint16_t *>(c.d_thread_infos);
    a.encoded = c.d_encoded;
    a.encoded_cap = c.encoded_cap;
    a.base_global_offset = c.base_global_offset;
    a.status = reinterpret_cast<uint32_t *>(slot);
    a.idx_offset = reinterpret_cast<uint32_t *>(c.d_idx_offset);
    a.stream_bytes = c.d_stream_bytes;
    a.result = c.d_result;
    a.max_polls = 0;
    a.force_order = 0;
    const int64_t chunks = (a.tiles + 1023) / 1024;
    KVC_REQUIRE((KVC_ENC_STATUS_WORDS + chunks) * 4 <= (int64_t)KVC_WS_SLOT_BYTES, "too many tiles (%lld) for one encode call",
                (long long)a.tiles);
    const unsigned wgs = (unsigned)((a.tiles + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG);
    const KvcStoreSource *src = c.src;
    const int is_k = c.is_k;
    KvcStoreArgs sa = {};
    if (src) {
        sa.e = a;
        sa.x = reinterpret_cast<const __half *>(src->x_f16);
        sa.B = (int)src->B;
        sa.H = (int)src->H;
        sa.D = (int)c.head_dim;
        sa.mask = src->mask;
        sa.eb = src->eb;
        sa.min_i8 = src->min_i8;
        sa.scale_f16 = reinterpret_cast<__half *>(src->scale_f16);
    }
    hipLaunchKernelGGL(kvc_encode_init_kernel, dim3(1), dim3(KVC_WAVE), 0, stream, a);
    // one pass (each wave counts, places and emits its tile) where the block_infos can serve as 64-bit status words.
    // From uint8 symbols there is no quantizing to save and the one-pass kernel runs at three waves per SIMD: measured on
    // MI355X at 65 536 / 49 152 tiles, K symbols encode 1.5 times and V symbols 1.6 times faster in one pass (which
    // fetches them through its LDS tile, whole token rows per load instruction) than in two.  So by default large
    // calls take the one pass (the option's values 2 and 3 send every call through it).
    const int one_pass = kvc_option(KVC_OPT_ENCODE_ONE_PASS);
    const bool symbols_in_one_pass = one_pass > 1 || (one_pass == 1 && a.tiles >= 8192);
    if ((src ? one_pass != 0 : symbols_in_one_pass) && ((uintptr_t)c.d_block_infos & 7) == 0 &&
        (a.tiles + KVC_ONCE_GROUP_TILES - 1) / KVC_ONCE_GROUP_TILES <= KVC_ONCE_MAX_GROUPS) {
        // how often a wave may find a word of its look-back not ready; -1 makes the call take the give-up path
        // (every wave still ends normally) so that tests can reach it from the host
        const int polls_opt = kvc_option(KVC_OPT_ENCODE_LOOKBACK_POLLS);
        a.max_polls = polls_opt < 0 ? 0 : polls_opt;
        a.force_order = polls_opt < 0;
        sa.e = a;
        const int front = !src ? 0 : is_k ? 1 : 2;
        const size_t lds = (size_t)(a.rows_per_codebook ? KVC_WAVES_PER_WG : 1) * 256 * sizeof(uint2) + (size_t)KVC_WAVES_PER_WG * KVC_ONCE_WAVE_BYTES;
        hipLaunchKernelGGL(kvc_encode_mark_kernel, dim3((unsigned)((a.tiles + KVC_WG - 1) / KVC_WG)), dim3(KVC_WG), 0, stream, a);
        // two tiles per wave (the look-back of the first hides behind the count of the second) where all tiles share
        // the codebook and there are enough of them to keep the chip full.  Longer runs would need the payloads of
        // more than one waiting tile in LDS.
        const int want = one_pass;
        int run = want == 1 ? (a.tiles >= 8192 ? 2 : 1) : want - 1;       // 2, 3: always one, two tiles per wave
        run = run < 1 ? 1 : run > 2 ? 2 : run;
        if (a.rows_per_codebook != 0) run = 1;
        const unsigned wgs1 = (unsigned)((a.tiles + (int64_t)run * KVC_WAVES_PER_WG - 1) / ((int64_t)run * KVC_WAVES_PER_WG));
        if (front == 0) {
            hipLaunchKernelGGL(kvc_encode_once_kernel<0>, dim3(wgs1), dim3(KVC_WG), lds, stream, sa, run);
            hipLaunchKernelGGL(kvc_encode_finish_kernel<0>, dim3(1), dim3(KVC_WG), 0, stream, sa);
        } else if (front == 1) {
            hipLaunchKernelGGL(kvc_encode_once_kernel<1>, dim3(wgs1), dim3(KVC_WG), lds, stream, sa, run);
            hipLaunchKernelGGL(kvc_encode_finish_kernel<1>, dim3(1), dim3(KVC_WG), 0, stream, sa);
        } else {
            hipLaunchKernelGGL(kvc_encode_once_kernel<2>, dim3(wgs1), dim3(KVC_WG), lds, stream, sa, run);
            hipLaunchKernelGGL(kvc_encode_finish_kernel<2>, dim3(1), dim3(KVC_WG), 0, stream, sa);
        }
        if (a.result || a.stream_bytes) hipLaunchKernelGGL(kvc_encode_publish_kernel, dim3(1), dim3(1), 0, stream, a);
        KVC_HIP(hipGetLastError());
        *slot_out = slot;
        return 0;
    }
    if (!src) hipLaunchKernelGGL(kvc_encode_count_kernel, dim3(wgs), dim3(KVC_WG), 0, stream, a);
    else if (is_k) hipLaunchKernelGGL(kvc_store_count_kernel<true>, dim3(wgs), dim3(KVC_WG), 0, stream, sa);
    else hipLaunchKernelGGL(kvc_store_count_kernel<false>, dim3(wgs), dim3(KVC_WG), 0, stream, sa);
    hipLaunchKernelGGL(kvc_encode_chunk_sum_kernel, dim3((unsigned)chunks), dim3(1024), 0, stream, a);
    hipLaunchKernelGGL(kvc_encode_scan_kernel, dim3((unsigned)chunks), dim3(1024), 0, stream, a);
    if (!src) hipLaunchKernelGGL(kvc_encode_emit_kernel, dim3(wgs), dim3(KVC_WG), 0, stream, a);
    else if (is_k) hipLaunchKernelGGL(kvc_store_emit_kernel<true>, dim3(wgs), dim3(KVC_WG), 0, stream, sa);
    else hipLaunchKernelGGL(kvc_store_emit_kernel<false>, dim3(wgs), dim3(KVC_WG), 0, stream, sa);
    if (a.result || a.stream_bytes) hipLaunchKernelGGL(kvc_encode_publish_kernel, dim3(1), dim3(1), 0, stream, a);
    KVC_HIP(hipGetLastError());
    *slot_out = slot;
    return 0;
}

static int kvc_entropy_encode(int is_k, const uint8_t *d_sym, int64_t tokens, int64_t stride,
                              const uint8_t *d_encode_table, int64_t encode_table_bytes, uint8_t *d_block_infos,
                              uint8_t *d_thread_infos, uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap,
                              uint32_t base_global_offset, int64_t head_dim, int64_t *h_total_bytes,
                              int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream_,
                              const KvcStoreSource *src = nullptr)
{
    hipStream_t stream = (hipStream_t)stream_;
    *h_total_bytes = 0;
    if (tokens == 0) {
        int64_t sizes[4];
        return kvc_calculate_buffer_size(tokens, stride, is_k, 0, head_dim, sizes);
    }
    KvcEncodeCall c = {};
    c.is_k = is_k;
    c.d_sym = d_sym;
    c.tokens = tokens;
    c.stride = stride;
    c.head_dim = head_dim;
    c.d_tables = d_encode_table;
    c.table_bytes = encode_table_bytes;
    c.d_block_infos = d_block_infos;
    c.d_thread_infos = d_thread_infos;
    c.d_idx_offset = d_idx_offset;
    c.d_encoded = d_encoded;
    c.encoded_cap = encoded_cap;
    c.base_global_offset = base_global_offset;
    c.src = src;
    void *slot;
    if (int rc = kvc_encode_launch(c, &slot, stream)) return rc;
    uint32_t h_status[4] = {0, 0, 0, 0};
    KVC_HIP(hipMemcpyAsync(h_status, slot, 16, hipMemcpyDeviceToHost, stream));
    KVC_HIP(hipStreamSynchronize(stream));   // the reference returns after cudaDeviceSynchronize (kernels.cu:957)
    if (int rc = kvc_encode_errors(h_status[1], h_status[0], encoded_cap)) return rc;
    *h_total_bytes = h_status[0];
    if (h_max_tile_bytes) *h_max_tile_bytes = h_status[2];
    if (h_max_stream_bytes) *h_max_stream_bytes = h_status[3];
    return 0;
}

extern "C" int kvc_k_entropy_encode(const uint8_t *d_sym, int64_t tokens, int64_t stride, const uint8_t *d_encode_table,
                                    int64_t encode_table_bytes, uint8_t *d_block_infos, uint8_t *d_thread_infos,
                                    uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap,
                                    uint32_t base_global_offset, int64_t head_num, int64_t head_dim,
                                    int64_t *h_total_bytes, int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream)
{
    (void)head_num;
    return kvc_entropy_encode(1, d_sym, tokens, stride, d_encode_table, encode_table_bytes, d_block_infos, d_thread_infos,
                              d_idx_offset, d_encoded, encoded_cap, base_global_offset, head_dim, h_total_bytes,
                              h_max_tile_bytes, h_max_stream_bytes, stream);
}

extern "C" int kvc_v_entropy_encode(const uint8_t *d_sym, int64_t tokens, int64_t stride, const uint8_t *d_encode_table,
                                    int64_t encode_table_bytes, uint8_t *d_block_infos, uint8_t *d_thread_infos,
                                    uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap,
                                    uint32_t base_global_offset, int64_t head_num, int64_t head_dim,
                                    int64_t *h_total_bytes, int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream)
{
    (void)head_num;
    return kvc_entropy_encode(0, d_sym, tokens, stride, d_encode_table, encode_table_bytes, d_block_infos, d_thread_infos,
                              d_idx_offset, d_encoded, encoded_cap, base_global_offset, head_dim, h_total_bytes,
                              h_max_tile_bytes, h_max_stream_bytes, stream);
}

// ---------------------------------------------------------------------------------------------------
// fused quantize + encode (no counterpart in the reference, which quantizes with ~8 fp16 tensor ops into a
// uint8 tensor and then encodes that: models/cache/kvcomp_encode.py:86-112)
// ---------------------------------------------------------------------------------------------------
extern "C" int kvc_store_fused_supported(int is_k, int quant_mask, int64_t batch, int64_t heads, int64_t head_dim)
{
    if (batch <= 0 || heads <= 0 || head_dim <= 0 || head_dim > 128 || head_dim % 8 != 0) return 0;
    if (is_k) return quant_mask == KVC_MASK_CHANNEL || quant_mask == KVC_MASK_K_BLOCK;
    if (quant_mask == KVC_MASK_V_TOKEN) return 1;
    return quant_mask == KVC_MASK_SIM_TOKEN && (heads * head_dim) % KVC_V_VEC_PER_BLK == 0;
}

extern "C" int kvc_store_fused(int is_k, const void *d_x_f16, int64_t tokens, int64_t batch, int64_t heads, int64_t head_dim,
                               int quant_mask, float eb, const uint8_t *d_encode_table, int64_t encode_table_bytes,
                               int8_t *d_min_i8, void *d_scale_f16, uint8_t *d_block_infos, uint8_t *d_thread_infos,
                               uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap, uint32_t base_global_offset,
                               int64_t *h_total_bytes, int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream)
{
    KVC_REQUIRE(kvc_store_fused_supported(is_k, quant_mask, batch, heads, head_dim),
                "fused store: unsupported layout (is_k %d, groups 0x%x, %lld heads x %lld)", is_k, quant_mask,
                (long long)heads, (long long)head_dim);
    KVC_REQUIRE(d_x_f16 != nullptr && d_min_i8 != nullptr && d_scale_f16 != nullptr, "NULL argument");
    KVC_REQUIRE(((uintptr_t)d_x_f16 & 3) == 0 && ((uintptr_t)d_scale_f16 & 1) == 0, "fp16 buffers are misaligned");
    KVC_REQUIRE(eb > 0.f, "error bound must be positive");
    const int64_t stride = batch * heads * head_dim;
    const int64_t bs = KVC_K_VEC_PER_BLK;                 // quantization block = 64 tokens in every supported layout
    KVC_REQUIRE(tokens >= 0 && tokens % (is_k ? KVC_K_VEC_PER_BLK : KVC_V_VEC_LEN) == 0, "token count must be whole tiles");
    if (tokens == 0) {
        if (h_total_bytes) *h_total_bytes = 0;
        return 0;
    }
    // every layout but per-channel K needs its group parameters before any tile can be quantized
    if (quant_mask != KVC_MASK_CHANNEL) {
        if (int rc = kvc_quant_params(d_x_f16, tokens / bs, bs, batch, heads, head_dim, quant_mask, eb, d_min_i8, d_scale_f16, stream))
            return rc;
    }
    KvcStoreSource src = {d_x_f16, batch, heads, quant_mask, eb, d_min_i8, d_scale_f16};
    return kvc_entropy_encode(is_k, nullptr, tokens, stride, d_encode_table, encode_table_bytes, d_block_infos, d_thread_infos,
                              d_idx_offset, d_encoded, encoded_cap, base_global_offset, head_dim, h_total_bytes,
                              h_max_tile_bytes, h_max_stream_bytes, stream, &src);
}

// ---------------------------------------------------------------------------------------------------
// encode without a host round trip: many codebooks per call, results left on the device (no counterpart in the
// reference, whose encoder copies its counters to the host and waits for the device on every call,
// kvcomp_cuda_extension/src/kernels.cu:950-965)
// ---------------------------------------------------------------------------------------------------
extern "C" int kvc_encode_async(const kvc_encode_job *job, void *stream)
{
    KVC_REQUIRE(job != nullptr, "NULL argument");
    KVC_REQUIRE(job->batch > 0 && job->heads > 0 && job->head_dim > 0 && job->tokens > 0, "empty geometry");
    KVC_REQUIRE(job->d_result != nullptr || job->d_stream_bytes != nullptr, "the call would leave no result anywhere");
    const int64_t stride = job->batch * job->heads * job->head_dim;
    KVC_REQUIRE(job->tokens % (job->is_k ? KVC_K_VEC_PER_BLK : KVC_V_VEC_LEN) == 0, "token count must be whole tiles");
    KvcEncodeCall c = {};
    c.is_k = job->is_k;
    c.d_sym = job->d_sym;
    c.tokens = job->tokens;
    c.stride = stride;
    c.head_dim = job->head_dim;
    c.d_tables = job->d_encode_tables;
    c.table_bytes = job->encode_table_bytes;
    c.table_stride = job->table_stride_bytes;
    c.rows_per_codebook = job->rows_per_codebook;
    c.d_meta = job->d_codebook_meta;
    c.d_block_infos = job->d_block_infos;
    c.d_thread_infos = job->d_thread_infos;
    c.d_idx_offset = nullptr;
    c.d_encoded = job->d_encoded;
    c.encoded_cap = job->encoded_cap;
    c.base_global_offset = job->base_global_offset;
    c.d_stream_bytes = job->d_stream_bytes;
    c.d_result = job->d_result;
    KvcStoreSource src = {job->d_x_f16, job->batch, job->heads, job->quant_mask, job->eb, job->d_min_i8, job->d_scale_f16};
    if (!job->d_sym) {
        KVC_REQUIRE(kvc_store_fused_supported(job->is_k, job->quant_mask, job->batch, job->heads, job->head_dim),
                    "fused store: unsupported layout (is_k %d, groups 0x%x, %lld heads x %lld)", job->is_k, job->quant_mask,
                    (long long)job->heads, (long long)job->head_dim);
        KVC_REQUIRE(job->d_x_f16 != nullptr && job->d_min_i8 != nullptr && job->d_scale_f16 != nullptr, "NULL argument");
        KVC_REQUIRE(((uintptr_t)job->d_x_f16 & 3) == 0 && ((uintptr_t)job->d_scale_f16 & 1) == 0, "fp16 buffers are misaligned");
        KVC_REQUIRE(job->eb > 0.f, "error bound must be positive");
        if (job->quant_mask != KVC_MASK_CHANNEL) {
            const int64_t bs = KVC_K_VEC_PER_BLK;
            if (int rc = kvc_quant_params(job->d_x_f16, job->tokens / bs, bs, job->batch, job->heads, job->head_dim, job->quant_mask,
                                          job->eb, job->d_min_i8, job->d_scale_f16, stream))
                return rc;
        }
        c.src = &src;
    }
    void *slot;
    return kvc_encode_launch(c, &slot, (hipStream_t)stream);
}

extern "C" int kvc_encode_result(const uint32_t *d_result, int64_t encoded_cap, int64_t *h_total_bytes, int64_t *h_max_tile_bytes,
                                 int64_t *h_max_stream_bytes, int64_t *h_tiles, void *stream)
{
    KVC_REQUIRE(d_result != nullptr, "NULL argument");
    uint32_t h[8] = {};
    KVC_HIP(hipMemcpyAsync(h, d_result, sizeof(h), hipMemcpyDeviceToHost, (hipStream_t)stream));
    KVC_HIP(hipStreamSynchronize((hipStream_t)stream));
    if (int rc = kvc_encode_errors(h[1], h[0], encoded_cap)) return rc;
    if (h_total_bytes) *h_total_bytes = h[0];
    if (h_max_tile_bytes) *h_max_tile_bytes = h[2];
    if (h_max_stream_bytes) *h_max_stream_bytes = h[3];
    if (h_tiles) *h_tiles = h[4];
    return 0;
}
