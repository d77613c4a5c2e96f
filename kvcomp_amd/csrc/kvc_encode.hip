// kvc_encode.hip -- bit-packed Huffman tile encoder.
//
// Replaces huffman_encode / v_huffman_encode and their launchers
// (kvcomp_cuda_extension/src/kernels.cu:181-235, 419-596, 919-1011).  One wave64 per tile, lane t owns
// vector t, as one 64-thread block does in the reference.  Three launches:
//
//   count  every lane adds up the code lengths of its vector; a wave prefix scan turns the 64 byte
//          counts into thread_infos and the tile's byte_num           (kernels.cu:448-465, 472-478)
//   scan   one workgroup turns the byte_nums into tile offsets, in tile order (the reference claims
//          offsets with a global atomic in arrival order, kernels.cu:474, which makes its stream
//          layout differ from run to run)
//   emit   every lane packs its codes MSB-first straight at its final position inside an LDS image
//          of the tile payload (words it shares with a neighbour lane are merged with LDS atomic OR),
//          and the wave copies the image out with aligned dword stores        (kernels.cu:181-235, 483-488)
//
// The symbols are read twice (1 B/symbol each) instead of once, which buys deterministic output
// and no per-lane scratch area: a lane's stream may be as long as the code allows.
#include "kvc_common.h"

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
    uint32_t base_global_offset;
    uint32_t *status;          // [0] total payload bytes, [1] error bits, [2] largest tile payload, [3] largest lane stream;
                               // from word KVC_ENC_STATUS_WORDS on: payload bytes of tiles 1024 j .. 1024 j + 1023
    uint32_t *idx_offset;      // {tiles, bytes}  (include/kernels.h:34-42)
};

constexpr int KVC_ENC_STATUS_WORDS = 16;            // status words in front of the per-1024-tile payload totals
constexpr uint32_t KVC_ENC_ERR_TILE_TOO_BIG = 1u;   // a tile payload exceeds 8191 bytes
constexpr uint32_t KVC_ENC_ERR_NO_CODE = 2u;        // a symbol without a code (length 0 or outside the table)
constexpr uint32_t KVC_ENC_ERR_CAPACITY = 4u;       // payload does not fit encoded_cap

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

__global__ void __launch_bounds__(KVC_WG) kvc_encode_count_kernel(KvcEncodeArgs a)
{
    __shared__ uint8_t s_len[256];
    __shared__ uint32_t s_err, s_longest;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) { s_err = 0; s_longest = 0; }
    {
        uint32_t len = 0;
        if (tid < a.table_entries) len = reinterpret_cast<const uint32_t *>(a.table)[2 * tid + 1];
        s_len[tid] = (uint8_t)(len > 32 ? 0 : len);
    }
    __syncthreads();
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    if (tile < a.tiles) {
        uint32_t v[32];
        kvc_load_vector(a, tile, lane, v);
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
        uint32_t err = bad ? KVC_ENC_ERR_NO_CODE : 0u;
        if (lane == KVC_WAVE - 1) {
            if (end > (uint32_t)KVC_MAX_TILE_BYTES) err |= KVC_ENC_ERR_TILE_TOO_BIG;
            // byte_num; the offset half of block_info is filled in by the scan kernel
            reinterpret_cast<uint32_t *>(a.block_infos + 8 * tile)[1] = end > 0xffffu ? 0xffffu : end;
        }
        if (err) atomicOr(&s_err, err);
        uint32_t longest = bytes;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)longest, off, 64);
            longest = o > longest ? o : longest;
        }
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
    uint32_t before = a.base_global_offset;
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
            if ((int64_t)total > a.encoded_cap) atomicOr(&a.status[1], KVC_ENC_ERR_CAPACITY);
            a.idx_offset[0] = (uint32_t)a.tiles;
            a.idx_offset[1] = total;
        }
    }
}

constexpr int KVC_IMAGE_WORDS = (KVC_MAX_TILE_BYTES + 3 + 3) / 4 + 1;   // payload + up to 3 leading bytes

__global__ void __launch_bounds__(KVC_WG) kvc_encode_emit_kernel(KvcEncodeArgs a)
{
    __shared__ uint2 s_table[256];
    __shared__ uint32_t s_image[KVC_WAVES_PER_WG][KVC_IMAGE_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    s_table[tid] = tid < a.table_entries ? reinterpret_cast<const uint2 *>(a.table)[tid] : make_uint2(0u, 0u);
    uint32_t *image = s_image[wave];
    for (int i = lane; i < KVC_IMAGE_WORDS; i += KVC_WAVE) image[i] = 0;
    __syncthreads();
    const int64_t tile = (int64_t)blockIdx.x * KVC_WAVES_PER_WG + wave;
    const bool active = tile < a.tiles;
    uint32_t off = 0, bn = 0, head = 0;
    if (active) {
        const uint32_t *bi = reinterpret_cast<const uint32_t *>(a.block_infos + 8 * tile);
        off = bi[0] - a.base_global_offset;
        bn = bi[1] & 0xffffu;
    }
    // a tile that does not fit (flagged by the earlier launches) is skipped, never written out of bounds
    const bool ok = active && bn <= (uint32_t)KVC_MAX_TILE_BYTES && (int64_t)off + bn <= a.encoded_cap;
    if (ok) {
        head = (uint32_t)((reinterpret_cast<uintptr_t>(a.encoded) + off) & 3u);
        uint32_t v[32];
        kvc_load_vector(a, tile, lane, v);
        const uint32_t start = lane ? (uint32_t)(a.thread_infos[tile * KVC_WAVE + lane - 1] >> 3) : 0u;
        const uint32_t bitpos = (head + start) * 8u;
        uint32_t w = bitpos >> 5, nacc = bitpos & 31u;
        uint64_t acc = 0;
        const int nd = a.vec_len >> 2;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            if (j < nd) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint2 e = s_table[(v[j] >> (8 * k)) & 0xffu];
                    const uint32_t len = e.y > 32u ? 0u : e.y;
                    acc = (acc << len) | e.x;
                    nacc += len;
                    if (nacc >= 32u) {
                        nacc -= 32u;
                        if (w < (uint32_t)KVC_IMAGE_WORDS) atomicOr(&image[w], kvc_bswap((uint32_t)(acc >> nacc)));
                        w++;
                        acc &= (1ull << nacc) - 1ull;
                    }
                }
            }
        }
        if (nacc > 0 && w < (uint32_t)KVC_IMAGE_WORDS) atomicOr(&image[w], kvc_bswap((uint32_t)(acc << (32u - nacc))));
    }
    __syncthreads();
    if (ok) {
        uint8_t *dst = a.encoded + off - head;                 // 4-byte aligned
        const uint32_t lo = head, hi = head + bn;              // valid byte range inside the image
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
}

static int kvc_entropy_encode(int is_k, const uint8_t *d_sym, int64_t tokens, int64_t stride,
                              const uint8_t *d_encode_table, int64_t encode_table_bytes, uint8_t *d_block_infos,
                              uint8_t *d_thread_infos, uint8_t *d_idx_offset, uint8_t *d_encoded, int64_t encoded_cap,
                              uint32_t base_global_offset, int64_t head_dim, int64_t *h_total_bytes,
                              int64_t *h_max_tile_bytes, int64_t *h_max_stream_bytes, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    int64_t sizes[4];
    if (int rc = kvc_calculate_buffer_size(tokens, stride, is_k, 0, head_dim, sizes)) return rc;
    *h_total_bytes = 0;
    if (tokens == 0) return 0;
    KVC_REQUIRE(head_dim % 8 == 0, "head_dim must be a multiple of 8");
    KVC_REQUIRE(encode_table_bytes > 0 && encode_table_bytes % 8 == 0 && encode_table_bytes <= 256 * 8,
                "encode table must hold 1..256 entries of 8 bytes");
    KVC_REQUIRE(((uintptr_t)d_encode_table & 7) == 0 && ((uintptr_t)d_block_infos & 3) == 0 &&
                ((uintptr_t)d_thread_infos & 1) == 0 && ((uintptr_t)d_idx_offset & 3) == 0 && ((uintptr_t)d_sym & 3) == 0,
                "encode buffers are misaligned");
    KVC_REQUIRE(stride % 4 == 0, "stride must be a multiple of 4");
    void *slot;
    if (int rc = kvc_workspace_slot(&slot)) return rc;
    KvcEncodeArgs a;
    a.sym = d_sym;
    a.stride = stride;
    a.is_k = is_k;
    a.vec_len = is_k ? (int)head_dim : KVC_V_TOKENS;
    a.cols = (int)(is_k ? stride / head_dim : stride / KVC_V_VEC_PER_BLK);
    a.tiles = sizes[0] / 8;
    a.table = d_encode_table;
    a.table_entries = (int)(encode_table_bytes / 8);
    a.block_infos = d_block_infos;
    a.thread_infos = reinterpret_cast<uint16_t *>(d_thread_infos);
    a.encoded = d_encoded;
    a.encoded_cap = encoded_cap;
    a.base_global_offset = base_global_offset;
    a.status = reinterpret_cast<uint32_t *>(slot);
    a.idx_offset = reinterpret_cast<uint32_t *>(d_idx_offset);
    const int64_t chunks = (a.tiles + 1023) / 1024;
    KVC_REQUIRE((KVC_ENC_STATUS_WORDS + chunks) * 4 <= (int64_t)KVC_WS_SLOT_BYTES, "too many tiles (%lld) for one encode call",
                (long long)a.tiles);
    KVC_HIP(hipMemsetAsync(slot, 0, (size_t)KVC_ENC_STATUS_WORDS * 4, stream));
    const unsigned wgs = (unsigned)((a.tiles + KVC_WAVES_PER_WG - 1) / KVC_WAVES_PER_WG);
    hipLaunchKernelGGL(kvc_encode_count_kernel, dim3(wgs), dim3(KVC_WG), 0, stream, a);
    hipLaunchKernelGGL(kvc_encode_chunk_sum_kernel, dim3((unsigned)chunks), dim3(1024), 0, stream, a);
    hipLaunchKernelGGL(kvc_encode_scan_kernel, dim3((unsigned)chunks), dim3(1024), 0, stream, a);
    hipLaunchKernelGGL(kvc_encode_emit_kernel, dim3(wgs), dim3(KVC_WG), 0, stream, a);
    KVC_HIP(hipGetLastError());
    uint32_t h_status[4] = {0, 0, 0, 0};
    KVC_HIP(hipMemcpyAsync(h_status, slot, 16, hipMemcpyDeviceToHost, stream));
    KVC_HIP(hipStreamSynchronize(stream));   // the reference returns after cudaDeviceSynchronize (kernels.cu:957)
    if (h_status[1] & KVC_ENC_ERR_NO_CODE) return kvc_fail(-3, "a symbol has no code in the encode table");
    if (h_status[1] & KVC_ENC_ERR_TILE_TOO_BIG)
        return kvc_fail(-3, "a tile encodes to more than %d bytes, which thread_info (u16) cannot address", KVC_MAX_TILE_BYTES);
    if (h_status[1] & KVC_ENC_ERR_CAPACITY)
        return kvc_fail(-3, "payload (%u bytes) does not fit the encoded_data buffer (%lld bytes)", h_status[0], (long long)encoded_cap);
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
