// kvc_tile.h -- device-side building blocks shared by the decoders: staging a tile payload in LDS and
// the table-driven, lock-step symbol decoder.
//
// One wave64 owns one tile: lane t owns stream t, exactly as one 64-thread block does in the reference
// (kvcomp_cuda_extension/src/kernels.cu:602-652).  Where the reference walks its decode tree one bit at
// a time (kernels.cu:237-291), a lane here peeks `lbits` stream bits, looks them up in an LDS table that
// yields (symbol, length), and shifts.  Every lane emits exactly one symbol per step, so the symbol index
// is uniform across the wave and the per-symbol operand of a fused kernel (q[i], p[t]*scale[t]) is a
// scalar, not a per-lane load.
#pragma once
#include "kvc_common.h"


struct KvcStreamArgs {
    const uint8_t *enc;            // concatenated tile payloads
    int64_t enc_bytes;
    const uint8_t *block_infos;    // 8 B per tile: {u32 offset; u16 byte_num; u16 pad}
    const uint16_t *thread_infos;  // 64 per tile: end_byte * 8 + pad_bits
    const uint32_t *luts;          // KVC_LUT_WORDS per codebook
    int rows_per_codebook;         // tile rows that share one codebook; 0 = one codebook for everything
    int cols;                      // tiles per tile row
    int tiles_per_wave;            // consecutive tiles (within a row) handled by one wave
    int vec_len;                   // symbols per lane stream
    int64_t stride;                // bytes (= symbols) per token in the [tokens, stride] symbol tensor
};

// Copy this workgroup's decode table into LDS.  Returns lbits/nlong/group through the header words.
__device__ __forceinline__ void kvc_load_lut(const uint32_t *__restrict__ lut_g, uint32_t *s_lut, int tid)
{
    const uint32_t lbits = lut_g[0], nlong = lut_g[2];
    if (tid < KVC_LUT_HEADER_WORDS) s_lut[tid] = lut_g[tid];
    for (uint32_t i = tid; i < 2 * nlong; i += KVC_WG) s_lut[KVC_LUT_HEADER_WORDS + i] = lut_g[KVC_LUT_HEADER_WORDS + i];
    const uint32_t *src = lut_g + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    uint32_t *dst = s_lut + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    for (uint32_t i = tid; i < (1u << lbits); i += KVC_WG) dst[i] = src[i];
}

// Stage the payload of `tile` into this wave's LDS area as big-endian 32-bit words (stream bit k of the
// staged area is bit 31 - (k & 31) of word k >> 5) and return the lane's first stream bit.
// Global reads are whole aligned 16-byte chunks that each contain at least one payload byte, so they
// never leave the pages the payload lives in.  Sizes are clamped so that a corrupt block_info or
// thread_info yields wrong symbols, never an out-of-bounds access.
__device__ __forceinline__ uint32_t kvc_stage_tile(const KvcStreamArgs &a, int64_t tile, uint32_t *stage, int lane)
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
    const uint4 *g = reinterpret_cast<const uint4 *>(base);
    uint4 *s = reinterpret_cast<uint4 *>(stage);
    for (uint32_t c = lane; c < nchunks; c += KVC_WAVE) {
        uint4 v = g[c];
        v.x = kvc_bswap(v.x);
        v.y = kvc_bswap(v.y);
        v.z = kvc_bswap(v.z);
        v.w = kvc_bswap(v.w);
        s[c] = v;
    }
    uint32_t start = lane ? (uint32_t)(a.thread_infos[tile * KVC_WAVE + lane - 1] >> 3) : 0u;
    if (start > bn) start = bn;
    return (head + start) * 8u;
}

// Decode n symbols (n a multiple of G) of this lane's stream, calling emit(i, symbol) for i = 0..n-1.
// G symbols are taken from one 32-bit window, which the table builder guarantees is enough
// (G * longest code <= 32).  SPILL adds the search through the codes that are longer than the table
// index; without it such bits decode as garbage but the loop still ends after n symbols.
template <int G, bool SPILL, class Emit>
__device__ __forceinline__ void kvc_decode_run(const uint32_t *stage, uint32_t &pos, const uint32_t *s_lut, int n, Emit &&emit)
{
    const uint32_t lshift = 32u - s_lut[0];
    const uint32_t nlong = SPILL ? s_lut[2] : 0u;
    const uint32_t *s_long = s_lut + KVC_LUT_HEADER_WORDS;
    const uint32_t *s_entry = s_lut + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    for (int i = 0; i < n; i += G) {
        uint32_t wi = pos >> 5;
        if (wi > (uint32_t)(KVC_STAGE_WORDS - 2)) wi = KVC_STAGE_WORDS - 2;
        const uint64_t w = ((uint64_t)stage[wi] << 32) | stage[wi + 1];
        uint32_t hi = (uint32_t)((w << (pos & 31u)) >> 32);
#pragma unroll
        for (int g = 0; g < G; g++) {
            uint32_t e = s_entry[hi >> lshift];
            uint32_t len = e & 0xffu;
            uint32_t sym = (e >> 8) & 0xffu;
            if (SPILL) {
                if (len == 0) {
                    len = 1;
                    sym = 0;
                    for (uint32_t j = 0; j < nlong; j++) {
                        const uint32_t c = s_long[2 * j], ls = s_long[2 * j + 1];
                        const uint32_t l = ls & 0xffu;
                        if (((hi ^ c) >> (32u - l)) == 0u) {
                            len = l;
                            sym = (ls >> 8) & 0xffu;
                            break;
                        }
                    }
                }
            }
            emit(i + g, sym);
            hi <<= (len & 31u);
            pos += len;
        }
    }
}

// Run `body.template operator()<G, SPILL>()` for the (group, spill) pair the table header asks for.
template <class Body>
__device__ __forceinline__ void kvc_dispatch_group(const uint32_t *s_lut, Body &&body)
{
    const uint32_t group = s_lut[3], nlong = s_lut[2];
    if (nlong == 0) {
        if (group >= 8) body.template operator()<8, false>();
        else if (group >= 4) body.template operator()<4, false>();
        else if (group >= 2) body.template operator()<2, false>();
        else body.template operator()<1, true>();
    } else {
        if (group >= 2) body.template operator()<2, true>();
        else body.template operator()<1, true>();
    }
}

// ---------------------------------------------------------------------------------------------------
// host side: geometry checks and launch shape shared by the decoders
// ---------------------------------------------------------------------------------------------------
static inline int kvc_fill_stream_args(KvcStreamArgs &s, const uint8_t *d_encoded, int64_t encoded_bytes,
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
    s.tiles_per_wave = 1;
    s.vec_len = is_k ? (int)head_dim : KVC_V_TOKENS;
    s.stride = stride;
    *rows_out = rows;
    return 0;
}

static inline dim3 kvc_grid(const KvcStreamArgs &s, int64_t rows)
{
    const int per_wg = KVC_WAVES_PER_WG * s.tiles_per_wave;
    return dim3((unsigned)((s.cols + per_wg - 1) / per_wg), (unsigned)rows);
}

