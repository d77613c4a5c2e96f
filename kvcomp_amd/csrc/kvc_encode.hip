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

// LDS traffic between the lanes of one wave needs no workgroup barrier (a wave's LDS operations complete in
// order); this keeps the compiler from moving accesses across the hand-over.
__device__ __forceinline__ void kvc_wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

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
                                                const uint2 *s_table, uint32_t *image, uint32_t head, bool short_codes)
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
            if (w < (uint32_t)KVC_IMAGE_WORDS) atomicOr(&image[w], kvc_bswap((uint32_t)(acc >> nacc)));
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
    if (nacc > 0 && w < (uint32_t)KVC_IMAGE_WORDS) atomicOr(&image[w], kvc_bswap((uint32_t)(acc << (32u - nacc))));
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
// Per-channel groups live entirely inside the tile: the count pass (PUBLISH) finds min / max itself, writes
// the group parameters and quantizes with exactly what it wrote (the minimum as int8), the emit pass reads
// them back, so the two passes always agree.
template <bool PUBLISH>
__device__ __forceinline__ void kvc_front_k(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, uint32_t (&v)[32])
{
    const int64_t stride = a.e.stride;
    const int D = a.D, RS = D + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const bool act = 2 * lane < D;
    const __half *p = a.x + (row * KVC_WAVE) * stride + col * D + (act ? 2 * lane : 0);
    auto lo = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu))); };
    auto hi = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); };
    KvcGroupParams g0, g1;
    if (a.mask == KVC_MASK_CHANNEL) {
        const int64_t g = row * stride + col * D + (act ? 2 * lane : 0);
        if (PUBLISH) {
            // two walks over the tile's rows (the second one finds them in the cache) keep the register count low
            float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
#pragma unroll 8
            for (int t = 0; t < KVC_WAVE; t++) {
                const uint32_t w = *reinterpret_cast<const uint32_t *>(p + t * stride);
                const float v0 = lo(w), v1 = hi(w);
                mn0 = fminf(mn0, v0); mx0 = fmaxf(mx0, v0);
                mn1 = fminf(mn1, v1); mx1 = fmaxf(mx1, v1);
            }
            g0 = kvc_group_params(mn0, mx0, a.eb);
            g1 = kvc_group_params(mn1, mx1, a.eb);
            const int8_t m0 = (int8_t)(int)g0.min_i, m1 = (int8_t)(int)g1.min_i;
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
        } else {
            g0 = kvc_stored_params(a, g);
            g1 = kvc_stored_params(a, g + 1);
        }
    } else {                                             // one pair per 64-token block (kernels.cu:771-772)
        g0 = g1 = kvc_stored_params(a, row);
    }
    if (act) {
#pragma unroll 8
        for (int t = 0; t < KVC_WAVE; t++) {
            const uint32_t w = *reinterpret_cast<const uint32_t *>(p + t * stride);
            const uint32_t s2 = (uint32_t)kvc_quant_one(lo(w), g0) | ((uint32_t)kvc_quant_one(hi(w), g1) << 8);
            *reinterpret_cast<uint16_t *>(s_sym + t * RS + 2 * lane) = (uint16_t)s2;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int nd = D >> 2;
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = j < nd ? *reinterpret_cast<const uint32_t *>(s_sym + lane * RS + 4 * j) : 0u;
}

// The count pass's variant: the lane keeps its two channels of all 64 tokens in registers (64 loads in flight, one walk
// over the tile instead of two), finds the groups' minima and maxima there, publishes the group parameters and quantizes.
__device__ __forceinline__ void kvc_front_k_once(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, uint32_t (&v)[32])
{
    const int64_t stride = a.e.stride;
    const int D = a.D, RS = D + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const bool act = 2 * lane < D;
    const __half *p = a.x + (row * KVC_WAVE) * stride + col * D + (act ? 2 * lane : 0);
    auto lo = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu))); };
    auto hi = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); };
    uint32_t raw[KVC_WAVE];
#pragma unroll
    for (int t = 0; t < KVC_WAVE; t++) raw[t] = *reinterpret_cast<const uint32_t *>(p + t * stride);
    KvcGroupParams g0, g1;
    if (a.mask == KVC_MASK_CHANNEL) {
        const int64_t g = row * stride + col * D + (act ? 2 * lane : 0);
        float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
#pragma unroll
        for (int t = 0; t < KVC_WAVE; t++) {
            const float v0 = lo(raw[t]), v1 = hi(raw[t]);
            mn0 = fminf(mn0, v0); mx0 = fmaxf(mx0, v0);
            mn1 = fminf(mn1, v1); mx1 = fmaxf(mx1, v1);
        }
        g0 = kvc_group_params(mn0, mx0, a.eb);
        g1 = kvc_group_params(mn1, mx1, a.eb);
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
    if (act) {
#pragma unroll
        for (int t = 0; t < KVC_WAVE; t++) {
            const uint32_t s2 = (uint32_t)kvc_quant_one(lo(raw[t]), g0) | ((uint32_t)kvc_quant_one(hi(raw[t]), g1) << 8);
            *reinterpret_cast<uint16_t *>(s_sym + t * RS + 2 * lane) = (uint16_t)s2;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int nd = D >> 2;
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = j < nd ? *reinterpret_cast<const uint32_t *>(s_sym + lane * RS + 4 * j) : 0u;
}

// V tile: 128 tokens x 64 flat channels.  While the tile is quantized, lane l owns channels 2 (l & 31), + 1 of
// tokens 64 (l >> 5) .. + 63 (one load instruction = two tokens' runs of 64 halves); four tokens' symbols of a
// channel are gathered in a register and written to LDS as one word of the [channel][token] tile, and lane c
// then reads channel c's vector.  Group parameters are per token (KVC_MASK_V_TOKEN) or per (token, batch
// entry) (KVC_MASK_SIM_TOKEN; the tile lies inside one batch entry); the wave first stages its 128 triples
// {scale, 1 / scale, min} in LDS.
__device__ __forceinline__ void kvc_front_v(const KvcStoreArgs &a, int64_t tile, int lane, uint8_t *s_sym, float *s_par,
                                            uint32_t (&v)[32])
{
    const int64_t stride = a.e.stride;
    constexpr int RS = KVC_V_TOKENS + 4;
    const int64_t row = tile / a.e.cols, col = tile - row * a.e.cols;
    const int pr = lane & 31, half = lane >> 5;
    const int64_t ch = col * KVC_WAVE + 2 * pr;
    const int64_t b = (col * KVC_WAVE) / ((int64_t)a.H * a.D);
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int t = lane + 64 * k;
        const int64_t tk = row * KVC_V_TOKENS + t;
        const KvcGroupParams g = kvc_stored_params(a, a.mask == KVC_MASK_V_TOKEN ? tk : tk * a.B + b);
        s_par[4 * t] = g.scale;
        s_par[4 * t + 1] = g.rcp;
        s_par[4 * t + 2] = g.min_i;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const __half *p = a.x + (row * KVC_V_TOKENS + 64 * half) * stride + ch;
#pragma unroll 2
    for (int jj = 0; jj < 16; jj++) {
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int t = 64 * half + 4 * jj + k;
            const uint32_t raw = *reinterpret_cast<const uint32_t *>(p + (int64_t)(4 * jj + k) * stride);
            KvcGroupParams g;
            g.scale = s_par[4 * t];
            g.rcp = s_par[4 * t + 1];
            g.min_i = s_par[4 * t + 2];
            g.min_h = __float2half_rn(g.min_i);
            const float v0 = __half2float(__ushort_as_half((unsigned short)(raw & 0xffffu)));
            const float v1 = __half2float(__ushort_as_half((unsigned short)(raw >> 16)));
            w0 |= (uint32_t)kvc_quant_one(v0, g) << (8 * k);
            w1 |= (uint32_t)kvc_quant_one(v1, g) << (8 * k);
        }
        *reinterpret_cast<uint32_t *>(s_sym + (2 * pr) * RS + 64 * half + 4 * jj) = w0;
        *reinterpret_cast<uint32_t *>(s_sym + (2 * pr + 1) * RS + 64 * half + 4 * jj) = w1;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < 32; j++) v[j] = *reinterpret_cast<const uint32_t *>(s_sym + lane * RS + 4 * j);
}

template <bool IS_K>
__global__ void __launch_bounds__(KVC_WG) kvc_store_count_kernel(KvcStoreArgs a)
{
    __shared__ uint8_t s_len[KVC_WAVES_PER_WG][256];
    __shared__ uint32_t s_err, s_longest;
    __shared__ __align__(16) uint8_t s_sym[KVC_WAVES_PER_WG][KVC_SYM_TILE_BYTES];
    __shared__ float s_par[IS_K ? 1 : KVC_WAVES_PER_WG][IS_K ? 4 : 4 * KVC_V_TOKENS];   // V: {scale, 1 / scale, min, -} per token
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) { s_err = 0; s_longest = 0; }
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (tile < a.e.tiles) kvc_load_len_table(a.e, tile, s_len[wave], lane);
    __syncthreads();
    if (tile < a.e.tiles) {
        uint32_t v[32];
        if (IS_K) kvc_front_k_once(a, tile, lane, s_sym[wave], v);
        else kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], v);
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
    __shared__ float s_par[IS_K ? 1 : KVC_WAVES_PER_WG][IS_K ? 4 : 4 * KVC_V_TOKENS];
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
    if (IS_K) kvc_front_k<false>(a, tile, lane, s_sym[wave], v);
    else kvc_front_v(a, tile, lane, s_sym[wave], s_par[wave], v);
    kvc_wave_lds_sync();                               // every lane holds its vector: the tile can be overwritten
    const uint32_t image_words = (p.head + p.bn + 3u) / 4u + 1u;
    for (uint32_t i = lane; i < image_words && i < (uint32_t)KVC_IMAGE_WORDS; i += KVC_WAVE) image[i] = 0;
    kvc_wave_lds_sync();
    kvc_pack_vector(a.e, kvc_stream_start(a.e, tile, lane), v, s_table[wave], image, p.head, s_short[wave] != 0u);
    kvc_wave_lds_sync();
    kvc_write_image(a.e, p, lane, image);
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
    if (int rc = kvc_workspace_slot(&slot)) return rc;
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
    const int64_t chunks = (a.tiles + 1023) / 1024;
    KVC_REQUIRE((KVC_ENC_STATUS_WORDS + chunks) * 4 <= (int64_t)KVC_WS_SLOT_BYTES, "too many tiles (%lld) for one encode call",
                (long long)a.tiles);
    const unsigned wgs = (unsigned)((a.tiles + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG);
    const KvcStoreSource *src = c.src;
    const int is_k = c.is_k;
    KvcStoreArgs sa;
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
