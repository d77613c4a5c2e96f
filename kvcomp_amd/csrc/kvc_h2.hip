// kvc_h2.hip -- the whole-tensor Huffman coder of the reference's utils/huffman.py:15-95 on the GPU.
//
// That function flattens a tensor row-major, builds one Huffman code over its values (min-heap on frequency
// only, a lone symbol gets the code '0') and returns the concatenation of the code bits as a bool tensor, one
// element per bit.  It is pure Python there (list appends per bit).  Here:
//   host   kvc_h2_codes          counts -> (code, length) per symbol, the tie-exact construction with the
//                                lone-symbol rule of utils/huffman.py:42-44
//   device kvc_h2_count_kernel   bits per chunk of 1024 symbols
//          kvc_h2_scan_kernel    exclusive prefix over the chunks (one workgroup)
//          kvc_h2_emit_kernel    each thread re-reads its 4 symbols, finds its bit offset by a workgroup scan
//                                and writes one byte (0 / 1) per code bit, most significant code bit first
#include "kvc_common.h"

constexpr int KVC_H2_SYMS_PER_THREAD = 4;
constexpr int KVC_H2_CHUNK = KVC_WG * KVC_H2_SYMS_PER_THREAD;   // 1024 symbols per workgroup

int kvc_huffman_codes_h2(const int64_t *counts, uint32_t code[256], uint32_t length[256]);   // kvc_host.hip

extern "C" int kvc_h2_codes(const int64_t *h_counts256, uint32_t *h_code256, uint32_t *h_length256)
{
    KVC_REQUIRE(h_counts256 && h_code256 && h_length256, "NULL argument");
    const int distinct = kvc_huffman_codes_h2(h_counts256, h_code256, h_length256);
    KVC_REQUIRE(distinct >= 0, "a Huffman code is longer than 32 bits");
    return 0;
}

__device__ __forceinline__ uint32_t kvc_h2_thread_bits(const uint8_t *__restrict__ sym, int64_t n, int64_t first,
                                                       const uint32_t *s_len, uint32_t (&len)[KVC_H2_SYMS_PER_THREAD],
                                                       uint32_t (&s)[KVC_H2_SYMS_PER_THREAD])
{
    uint32_t bits = 0;
#pragma unroll
    for (int j = 0; j < KVC_H2_SYMS_PER_THREAD; j++) {
        len[j] = 0;
        s[j] = 0;
        if (first + j < n) {
            s[j] = sym[first + j];
            len[j] = s_len[s[j]];
        }
        bits += len[j];
    }
    return bits;
}

__global__ void __launch_bounds__(KVC_WG)
kvc_h2_count_kernel(const uint8_t *__restrict__ sym, int64_t n, const uint32_t *__restrict__ length256,
                    unsigned long long *__restrict__ chunk_bits)
{
    __shared__ uint32_t s_len[256];
    __shared__ uint32_t s_total;
    s_len[threadIdx.x] = length256[threadIdx.x];
    if (threadIdx.x == 0) s_total = 0;
    __syncthreads();
    uint32_t len[KVC_H2_SYMS_PER_THREAD], s[KVC_H2_SYMS_PER_THREAD];
    const int64_t first = ((int64_t)blockIdx.x * KVC_WG + threadIdx.x) * KVC_H2_SYMS_PER_THREAD;
    const uint32_t bits = kvc_h2_thread_bits(sym, n, first, s_len, len, s);
    const uint32_t wave_bits = kvc_wave_inclusive_scan(bits, threadIdx.x & 63);
    if ((threadIdx.x & 63) == 63) atomicAdd(&s_total, wave_bits);
    __syncthreads();
    if (threadIdx.x == 0) chunk_bits[blockIdx.x] = s_total;
}

// in place: chunk_bits[c] <- bits before chunk c; chunk_bits[chunks] <- total
__global__ void __launch_bounds__(1024) kvc_h2_scan_kernel(unsigned long long *chunk_bits, int64_t chunks)
{
    __shared__ unsigned long long s_wave[16];
    __shared__ unsigned long long s_carry;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) s_carry = 0;
    __syncthreads();
    for (int64_t base = 0; base < chunks; base += 1024) {
        const int64_t c = base + tid;
        const unsigned long long mine = c < chunks ? chunk_bits[c] : 0ull;
        unsigned long long incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const unsigned long long t = __shfl_up(incl, off, 64);
            if (lane >= off) incl += t;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        unsigned long long before = s_carry;
        for (int w = 0; w < wave; w++) before += s_wave[w];
        if (c < chunks) chunk_bits[c] = before + incl - mine;
        __syncthreads();
        if (tid == 1023) s_carry = before + incl;
        __syncthreads();
    }
    if (tid == 0) chunk_bits[chunks] = s_carry;
}

__global__ void __launch_bounds__(KVC_WG)
kvc_h2_emit_kernel(const uint8_t *__restrict__ sym, int64_t n, const uint32_t *__restrict__ code256,
                   const uint32_t *__restrict__ length256, const unsigned long long *__restrict__ chunk_bits,
                   uint8_t *__restrict__ bits_out)
{
    __shared__ uint32_t s_len[256], s_code[256];
    __shared__ uint32_t s_wave[KVC_WAVES_PER_WG];
    s_len[threadIdx.x] = length256[threadIdx.x];
    s_code[threadIdx.x] = code256[threadIdx.x];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t len[KVC_H2_SYMS_PER_THREAD], s[KVC_H2_SYMS_PER_THREAD];
    const int64_t first = ((int64_t)blockIdx.x * KVC_WG + threadIdx.x) * KVC_H2_SYMS_PER_THREAD;
    const uint32_t bits = kvc_h2_thread_bits(sym, n, first, s_len, len, s);
    const uint32_t incl = kvc_wave_inclusive_scan(bits, lane);
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = incl - bits;
    for (int w = 0; w < wave; w++) before += s_wave[w];
    uint8_t *o = bits_out + chunk_bits[blockIdx.x] + before;
#pragma unroll
    for (int j = 0; j < KVC_H2_SYMS_PER_THREAD; j++) {
        const uint32_t c = s_code[s[j]];
        for (uint32_t b = 0; b < len[j]; b++) *o++ = (uint8_t)((c >> (len[j] - 1 - b)) & 1u);
    }
}

extern "C" int64_t kvc_h2_scratch_bytes(int64_t n)
{
    if (n < 0) return 0;
    const int64_t chunks = (n + KVC_H2_CHUNK - 1) / KVC_H2_CHUNK;
    return (chunks + 1) * 8 + 2 * 256 * 4;
}

extern "C" int kvc_h2_encode(const uint8_t *d_sym, int64_t n, const uint32_t *h_code256, const uint32_t *h_length256,
                             uint8_t *d_bits, int64_t bits_cap, void *d_scratch, int64_t scratch_bytes,
                             int64_t *h_total_bits, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(h_total_bits != nullptr && h_code256 != nullptr && h_length256 != nullptr, "NULL argument");
    *h_total_bits = 0;
    if (n == 0) return 0;
    KVC_REQUIRE(n > 0 && d_sym != nullptr, "bad input");
    KVC_REQUIRE(d_scratch != nullptr && ((uintptr_t)d_scratch & 7) == 0 && scratch_bytes >= kvc_h2_scratch_bytes(n),
                "scratch needs %lld bytes, 8-byte aligned", (long long)kvc_h2_scratch_bytes(n));
    for (int s = 0; s < 256; s++) KVC_REQUIRE(h_length256[s] <= 32, "code length above 32");
    const int64_t chunks = (n + KVC_H2_CHUNK - 1) / KVC_H2_CHUNK;
    KVC_REQUIRE(chunks <= 0x7fffffff, "input too long for one call");
    unsigned long long *chunk_bits = reinterpret_cast<unsigned long long *>(d_scratch);
    uint32_t *d_code = reinterpret_cast<uint32_t *>(chunk_bits + chunks + 1), *d_len = d_code + 256;
    KVC_HIP(hipMemcpyAsync(d_code, h_code256, 1024, hipMemcpyHostToDevice, stream));
    KVC_HIP(hipMemcpyAsync(d_len, h_length256, 1024, hipMemcpyHostToDevice, stream));
    hipLaunchKernelGGL(kvc_h2_count_kernel, dim3((unsigned)chunks), dim3(KVC_WG), 0, stream, d_sym, n, d_len, chunk_bits);
    hipLaunchKernelGGL(kvc_h2_scan_kernel, dim3(1), dim3(1024), 0, stream, chunk_bits, chunks);
    KVC_HIP(hipGetLastError());
    unsigned long long total = 0;
    KVC_HIP(hipMemcpyAsync(&total, chunk_bits + chunks, 8, hipMemcpyDeviceToHost, stream));
    KVC_HIP(hipStreamSynchronize(stream));
    *h_total_bits = (int64_t)total;
    if (d_bits == nullptr) return 0;                 // size query
    KVC_REQUIRE((int64_t)total <= bits_cap, "the bitstream has %lld bits, the buffer holds %lld", (long long)total,
                (long long)bits_cap);
    hipLaunchKernelGGL(kvc_h2_emit_kernel, dim3((unsigned)chunks), dim3(KVC_WG), 0, stream, d_sym, n, d_code, d_len,
                       chunk_bits, d_bits);
    return kvc_check_hip(hipGetLastError(), "kvc_h2_emit_kernel launch");
}
