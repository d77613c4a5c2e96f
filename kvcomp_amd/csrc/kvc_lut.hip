// kvc_lut.hip -- turns a decode tree (the reference's 3-byte node array, src/huffman.cpp:229-252, or
// the wide 5-byte variant) into the table-driven form the decoders use.
//
// One 256-thread workgroup per codebook:
//   1. unpack the nodes into LDS (leaf flag, two children / the symbol);
//   2. record each node's parent and incoming bit, then every leaf walks up to the root: that gives its
//      code length, hence lmax, and the left-aligned code of every "long" code (length > lbits);
//   3. every table index walks down from the root along its own bits until it meets a leaf.
// A malformed tree (child index out of range, cycles) cannot hang or fault: walks are bounded by 32
// steps and indices are range-checked; the affected entries stay 0 (= "no code").
#include "kvc_common.h"

__global__ void __launch_bounds__(KVC_WG)
kvc_build_lut_kernel(const uint8_t *__restrict__ trees, int64_t tree_stride, int tree_bytes, int node_bytes,
                     uint32_t *__restrict__ luts)
{
    __shared__ int16_t s_child[2][KVC_TREE_MAX_NODES];
    __shared__ int16_t s_parent[KVC_TREE_MAX_NODES];
    __shared__ uint8_t s_leaf[KVC_TREE_MAX_NODES];
    __shared__ uint8_t s_bit[KVC_TREE_MAX_NODES];
    __shared__ uint32_t s_lmax, s_nlong;
    __shared__ float s_avg;   // sum over leaves of len * 2^-len: the mean code length if the code is well matched
    __shared__ uint32_t s_symbits;   // OR over the symbols' fp16 patterns

    const int tid = threadIdx.x;
    const uint8_t *tree = trees + (int64_t)blockIdx.x * tree_stride;
    uint32_t *lut = luts + (int64_t)blockIdx.x * KVC_LUT_WORDS;
    int n_nodes = tree_bytes / node_bytes;
    if (n_nodes > KVC_TREE_MAX_NODES) n_nodes = KVC_TREE_MAX_NODES;

    if (tid == 0) { s_lmax = 0; s_nlong = 0; s_avg = 0.f; s_symbits = 0; }
    for (int n = tid; n < KVC_TREE_MAX_NODES; n += KVC_WG) {
        int leaf = 0, a = -1, b = -1;
        if (n < n_nodes) {
            const uint8_t *p = tree + (int64_t)n * node_bytes;
            leaf = p[0] != 0;
            if (node_bytes == KVC_TREE_I8) {
                a = (int8_t)p[1];
                b = (int8_t)p[2];
            } else {
                a = (int16_t)(p[1] | (p[2] << 8));
                b = (int16_t)(p[3] | (p[4] << 8));
            }
            if (leaf) { a &= 0xff; b = a; }   // symbol value 0..255 (the int8 form stores it sign-wrapped)
        }
        s_leaf[n] = (uint8_t)leaf;
        s_child[0][n] = (int16_t)a;
        s_child[1][n] = (int16_t)b;
        s_parent[n] = -1;
        s_bit[n] = (uint8_t)(n & 1);          // nodes 0 / 1 hang off the implicit root by bit 0 / 1
    }
    __syncthreads();
    for (int n = tid; n < n_nodes; n += KVC_WG) {
        if (s_leaf[n]) continue;
        for (int bit = 0; bit < 2; bit++) {
            int c = s_child[bit][n];
            if (c >= 2 && c < n_nodes) { s_parent[c] = (int16_t)n; s_bit[c] = (uint8_t)bit; }
        }
    }
    __syncthreads();
    // leaf -> root: length and code (bits arrive last-first)
    uint32_t my_len[KVC_TREE_MAX_NODES / KVC_WG], my_code[KVC_TREE_MAX_NODES / KVC_WG];
#pragma unroll
    for (int k = 0; k < KVC_TREE_MAX_NODES / KVC_WG; k++) {
        int n = tid + k * KVC_WG;
        my_len[k] = 0;
        my_code[k] = 0;
        if (n < n_nodes && s_leaf[n]) {
            uint32_t len = 0, code = 0;
            int cur = n;
            while (len < 33) {
                code |= (uint32_t)s_bit[cur] << (len & 31);
                len++;
                int par = s_parent[cur];
                if (par < 0) break;
                cur = par;
            }
            // a valid chain ends at node 0 or 1; anything else (orphan, over-long) is ignored
            if (len <= 32 && cur < 2) {
                my_len[k] = len;
                my_code[k] = code;
                atomicMax(&s_lmax, len);
                atomicAdd(&s_avg, (float)len * exp2f(-(float)len));
                atomicOr(&s_symbits, (uint32_t)__half_as_ushort(__float2half_rn((float)(s_child[0][n] & 0xff))));
            }
        }
    }
    __syncthreads();
    const uint32_t lmax = s_lmax;
    const uint32_t lbits = lmax == 0 ? 1u : (lmax < (uint32_t)KVC_LUT_MAX_BITS ? lmax : (uint32_t)KVC_LUT_MAX_BITS);
#pragma unroll
    for (int k = 0; k < KVC_TREE_MAX_NODES / KVC_WG; k++) {
        if (my_len[k] > lbits) {
            uint32_t slot = atomicAdd(&s_nlong, 1u);
            if (slot < (uint32_t)KVC_LUT_MAX_LONG) {
                int n = tid + k * KVC_WG;
                lut[KVC_LUT_HEADER_WORDS + 2 * slot] = my_code[k] << (32 - my_len[k]);
                lut[KVC_LUT_HEADER_WORDS + 2 * slot + 1] = my_len[k] | ((uint32_t)(s_child[0][n] & 0xff) << 8);
            }
        }
    }
    // table entries: walk down along the index bits
    uint32_t *entries = lut + KVC_LUT_HEADER_WORDS + KVC_LUT_LONG_WORDS;
    for (uint32_t idx = tid; idx < (1u << lbits); idx += KVC_WG) {
        uint32_t e = 0;
        int cur = (int)((idx >> (lbits - 1)) & 1u);
        for (uint32_t depth = 1; depth <= lbits; depth++) {
            if (cur < 0 || cur >= n_nodes) break;
            if (s_leaf[cur]) { e = depth | ((uint32_t)(s_child[0][cur] & 0xff) << 8); break; }
            if (depth == lbits) break;
            cur = s_child[(idx >> (lbits - 1 - depth)) & 1u][cur];
        }
        entries[idx] = e;
    }
    // fused-kernel entries: the index bits are the stream bits in arrival order from bit 0 up (the fused
    // kernels keep their window least-significant-bit first), so walk with bit j of the index at depth j
    for (uint32_t idx = tid; idx < (1u << lbits); idx += KVC_WG) {
        uint32_t e = 1u;                       // no code / code longer than the index: "symbol 0, length 1"
        int cur = (int)(idx & 1u);
        for (uint32_t depth = 1; depth <= lbits; depth++) {
            if (cur < 0 || cur >= n_nodes) break;
            if (s_leaf[cur]) { e = __float_as_uint((float)(s_child[0][cur] & 0xff)) | depth; break; }
            if (depth == lbits) break;
            cur = s_child[(idx >> depth) & 1u][cur];
        }
        lut[KVC_LUT_FENTRY_OFFSET + idx] = e;
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t nlong = s_nlong < (uint32_t)KVC_LUT_MAX_LONG ? s_nlong : (uint32_t)KVC_LUT_MAX_LONG;
        uint32_t group = lmax <= 4 ? 8u : lmax <= 8 ? 4u : lmax <= 16 ? 2u : 1u;
        lut[0] = lbits;
        lut[1] = lmax;
        lut[2] = nlong;
        lut[3] = group;
        const bool roomy = s_avg <= 5.5f;
        const bool roomy8 = lmax == 4 && s_avg <= 2.75f;
        // symbols that a 30-bit window is sure to hold (30 / lmax, at most 8); more where the average code is short
        // enough for the window to overflow rarely (lut[5] = 1: the kernel checks and falls back)
        lut[4] = (lmax <= 3 || roomy8) ? 8u : lmax <= 7 ? 30u / lmax : roomy ? 4u : 2u;
        lut[5] = (roomy8 || (lmax > 7 && roomy)) ? 1u : 0u;
        lut[6] = s_symbits;       // low bits clear in every symbol's fp16 pattern: room for lengths in a packed entry
        lut[7] = 0;
    }
}

int kvc_launch_build_lut(const uint8_t *d_tree, int64_t tree_bytes, int tree_format, uint32_t *d_lut,
                         int n_codebooks, int64_t tree_stride_bytes, hipStream_t stream)
{
    KVC_REQUIRE(tree_format == KVC_TREE_I8 || tree_format == KVC_TREE_I16, "unknown tree format %d", tree_format);
    KVC_REQUIRE(tree_bytes >= 2 * tree_format && tree_bytes % tree_format == 0,
                "decode tree size %lld is not a whole number (>= 2) of %d-byte nodes", (long long)tree_bytes, tree_format);
    KVC_REQUIRE(tree_bytes / tree_format <= KVC_TREE_MAX_NODES, "decode tree has more than %d nodes", KVC_TREE_MAX_NODES);
    hipLaunchKernelGGL(kvc_build_lut_kernel, dim3(n_codebooks), dim3(KVC_WG), 0, stream, d_tree, tree_stride_bytes,
                       (int)tree_bytes, tree_format, d_lut);
    return kvc_check_hip(hipGetLastError(), "kvc_build_lut_kernel launch");
}
