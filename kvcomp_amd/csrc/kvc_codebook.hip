// kvc_codebook.hip -- Huffman codebooks built on the device, many at a time, with no host round trip.
//
//   kvc_histogram_chunks       <- torch::bincount per input of build_codebook (src/huffman.cpp:105-109): one
//                                 256-bin histogram per equal-sized chunk of a symbol tensor (a chunk = the tile
//                                 rows that share a codebook)
//   kvc_build_codebook_device  <- gen_huffman_codes + build_codebook (src/huffman.cpp:34-157, 166-187, 229-252):
//                                 counts -> {code, length} per symbol -> encode table and decode tree, the same
//                                 bytes kvc_build_codebook_host returns
//
// The reference merges nodes out of a std::priority_queue that compares frequencies only, so which of several
// equal-frequency nodes leaves first is decided by the array-heap algorithm (push: append, sift up while strictly
// smaller than the parent; pop: move the root hole down towards the smaller child, right child on a tie, drop the
// former last element into the hole, sift it up).  That algorithm is sequential; here one lane per codebook runs
// it in LDS (about 0.3 ms for 256 symbols) while the other codebooks of the launch run beside it on other
// workgroups, and the whole workgroup then writes the tables.
#include "kvc_common.h"

constexpr int KVC_CB_THREADS = 64;
constexpr int KVC_CB_ENCODE_BYTES = 256 * 8;          // {u32 code; u32 length} for every possible symbol
constexpr int KVC_CB_STATUS_FEW = 1;                  // fewer than two distinct symbols
constexpr int KVC_CB_STATUS_LONG = 2;                 // a code is longer than 32 bits
constexpr int KVC_CB_STATUS_INT8 = 4;                 // not representable in the 3-byte (int8) tree

static int kvc_cb_tree_nodes(int tree_format) { return tree_format == KVC_TREE_I8 ? 128 : KVC_TREE_MAX_NODES; }

extern "C" int64_t kvc_codebook_tree_capacity(int tree_format)
{
    if (tree_format != KVC_TREE_I8 && tree_format != KVC_TREE_I16) return 0;
    return (int64_t)kvc_cb_tree_nodes(tree_format) * tree_format;
}

namespace {
// the frequency heap of the construction, in LDS
struct KvcDevHeap {
    int16_t *h;
    const int64_t *f;
    int n;
    __device__ bool less(int a, int b) const { return f[a] < f[b]; }
    __device__ void push(int x)
    {
        int pos = n++;
        while (pos > 0) {
            const int par = (pos - 1) >> 1;
            if (!less(x, h[par])) break;
            h[pos] = h[par];
            pos = par;
        }
        h[pos] = (int16_t)x;
    }
    __device__ int pop()
    {
        const int last = h[--n];
        if (n == 0) return last;
        const int top = h[0];
        int pos = 0, child = 1;
        while (child < n) {
            const int right = child + 1;
            if (right < n && !less(h[child], h[right])) child = right;
            h[pos] = h[child];
            pos = child;
            child = 2 * pos + 1;
        }
        while (pos > 0) {
            const int par = (pos - 1) >> 1;
            if (!less(last, h[par])) break;
            h[pos] = h[par];
            pos = par;
        }
        h[pos] = (int16_t)last;
        return top;
    }
};
}  // namespace

// One workgroup per codebook.  meta[4 * cb ..] = {smallest symbol ("shift"), encode table bytes, decode tree
// bytes, status}; with a non-zero status both sizes are 0 and the tables are filled with "no code".
__global__ void __launch_bounds__(KVC_CB_THREADS)
kvc_build_codebook_kernel(const int64_t *__restrict__ counts_all, int tree_format, int tree_nodes_cap,
                          uint8_t *__restrict__ encode_tables, uint8_t *__restrict__ decode_trees, int32_t *__restrict__ meta)
{
    __shared__ int64_t s_f[512];
    __shared__ int16_t s_left[512], s_right[512], s_sym[512];
    __shared__ int16_t s_heap[256];
    __shared__ uint32_t s_code[256];
    __shared__ uint8_t s_len[256];
    __shared__ int16_t s_stack_node[264];
    __shared__ uint64_t s_stack_code[264];
    __shared__ uint8_t s_stack_len[264];
    __shared__ uint8_t s_tleaf[KVC_TREE_MAX_NODES];
    __shared__ int16_t s_tchild[2][KVC_TREE_MAX_NODES];
    __shared__ int s_status, s_mn, s_mx, s_tnodes;
    const int tid = threadIdx.x;
    const int64_t cb = blockIdx.x;
    const int64_t *counts = counts_all + cb * 256;
    for (int s = tid; s < 256; s += KVC_CB_THREADS) {
        s_code[s] = 0;
        s_len[s] = 0;
    }
    __syncthreads();
    if (tid == 0) {
        int status = 0, nn = 0, mn = 255, mx = 0;
        KvcDevHeap heap = {s_heap, s_f, 0};
        // leaves in ascending symbol order (huffman.cpp:44-52)
        for (int s = 0; s < 256; s++) {
            const int64_t c = counts[s];
            if (c > 0) {
                s_f[nn] = c;
                s_left[nn] = s_right[nn] = -1;
                s_sym[nn] = (int16_t)s;
                heap.push(nn);
                nn++;
                if (s < mn) mn = s;
                if (s > mx) mx = s;
            }
        }
        if (nn < 2) {
            status |= KVC_CB_STATUS_FEW;
        } else {
            // merge the two smallest until one node is left; first pop = left = bit 0 (huffman.cpp:54-70)
            while (heap.n > 1) {
                const int a = heap.pop();
                const int b = heap.pop();
                s_f[nn] = s_f[a] + s_f[b];
                s_left[nn] = (int16_t)a;
                s_right[nn] = (int16_t)b;
                s_sym[nn] = -1;
                heap.push(nn);
                nn++;
            }
            // codes: walk down from the root
            int sp = 0;
            s_stack_node[0] = s_heap[0];
            s_stack_code[0] = 0;
            s_stack_len[0] = 0;
            sp = 1;
            while (sp > 0) {
                sp--;
                const int node = s_stack_node[sp];
                const uint64_t code = s_stack_code[sp];
                const int len = s_stack_len[sp];
                if (s_left[node] < 0) {
                    if (len > 32) {
                        status |= KVC_CB_STATUS_LONG;
                    } else {
                        s_code[s_sym[node]] = (uint32_t)code;
                        s_len[s_sym[node]] = (uint8_t)len;
                    }
                } else if (len >= 63) {
                    status |= KVC_CB_STATUS_LONG;
                } else {
                    s_stack_node[sp] = s_right[node];
                    s_stack_code[sp] = (code << 1) | 1u;
                    s_stack_len[sp] = (uint8_t)(len + 1);
                    sp++;
                    s_stack_node[sp] = s_left[node];
                    s_stack_code[sp] = code << 1;
                    s_stack_len[sp] = (uint8_t)(len + 1);
                    sp++;
                }
            }
        }
        // decode tree: symbols in ascending order, nodes appended on demand; nodes 0 / 1 hang off the implicit
        // root (huffman.cpp:229-252)
        int tn = 2;
        s_tleaf[0] = s_tleaf[1] = 0;
        s_tchild[0][0] = s_tchild[1][0] = s_tchild[0][1] = s_tchild[1][1] = -1;
        if (status == 0) {
            for (int s = 0; s < 256 && status == 0; s++) {
                const int len = s_len[s];
                if (len == 0) continue;
                const uint32_t code = s_code[s];
                int idx = -1, last = -1;
                for (int i = 0; i < len; i++) {
                    const int bit = (int)((code >> (len - 1 - i)) & 1u);
                    idx = (idx == -1) ? bit : s_tchild[bit][idx];
                    if (idx == -1) {
                        if (tn >= KVC_TREE_MAX_NODES) { status |= KVC_CB_STATUS_LONG; break; }   // cannot happen for a prefix code
                        idx = tn++;
                        s_tleaf[idx] = 0;
                        s_tchild[0][idx] = s_tchild[1][idx] = -1;
                        s_tchild[bit][last] = (int16_t)idx;
                    }
                    last = idx;
                }
                if (status) break;
                s_tleaf[idx] = 1;
                s_tchild[0][idx] = s_tchild[1][idx] = (int16_t)s;
            }
            if (tree_format == KVC_TREE_I8 && (tn > 128 || mx > 127)) status |= KVC_CB_STATUS_INT8;
        }
        s_status = status;
        s_mn = mn;
        s_mx = mx;
        s_tnodes = tn;
    }
    __syncthreads();
    const int status = s_status, mn = s_mn, mx = s_mx, tn = s_tnodes;
    // encode table: entry i <-> symbol shift + i, absent symbols {0, 0} (huffman.cpp:166-187)
    uint32_t *enc = reinterpret_cast<uint32_t *>(encode_tables + cb * KVC_CB_ENCODE_BYTES);
    for (int w = tid; w < KVC_CB_ENCODE_BYTES / 4; w += KVC_CB_THREADS) {
        const int s = mn + (w >> 1);
        uint32_t v = 0;
        if (status == 0 && s <= mx && s_len[s] != 0) v = (w & 1) ? (uint32_t)s_len[s] : s_code[s];
        enc[w] = v;
    }
    // decode tree, padded to its capacity with childless inner nodes (never reached from the root)
    uint8_t *tree = decode_trees + cb * (int64_t)tree_nodes_cap * tree_format;
    for (int n = tid; n < tree_nodes_cap; n += KVC_CB_THREADS) {
        const bool live = status == 0 && n < tn;
        const int leaf = live ? s_tleaf[n] : 0;
        const int a = live ? s_tchild[0][n] : -1, b = live ? s_tchild[1][n] : -1;
        uint8_t *p = tree + (int64_t)n * tree_format;
        p[0] = (uint8_t)leaf;
        if (tree_format == KVC_TREE_I8) {
            p[1] = (uint8_t)(int8_t)a;
            p[2] = (uint8_t)(int8_t)b;
        } else {
            p[1] = (uint8_t)(a & 0xff);
            p[2] = (uint8_t)((a >> 8) & 0xff);
            p[3] = (uint8_t)(b & 0xff);
            p[4] = (uint8_t)((b >> 8) & 0xff);
        }
    }
    if (tid == 0) {
        meta[4 * cb] = mn <= mx ? mn : 0;
        meta[4 * cb + 1] = status == 0 ? (mx - mn + 1) * 8 : 0;
        meta[4 * cb + 2] = status == 0 ? tn * tree_format : 0;
        meta[4 * cb + 3] = status;
    }
}

extern "C" int kvc_build_codebook_device(const int64_t *d_counts, int64_t n_codebooks, int tree_format,
                                         uint8_t *d_encode_tables, uint8_t *d_decode_trees, int32_t *d_meta, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    KVC_REQUIRE(tree_format == KVC_TREE_I8 || tree_format == KVC_TREE_I16, "unknown tree format %d", tree_format);
    KVC_REQUIRE(n_codebooks >= 0 && n_codebooks < (1ll << 31), "bad codebook count %lld", (long long)n_codebooks);
    if (n_codebooks == 0) return 0;
    KVC_REQUIRE(d_counts && d_encode_tables && d_decode_trees && d_meta, "NULL argument");
    KVC_REQUIRE(((uintptr_t)d_counts & 7) == 0 && ((uintptr_t)d_encode_tables & 7) == 0 && ((uintptr_t)d_meta & 3) == 0,
                "codebook buffers are misaligned");
    hipLaunchKernelGGL(kvc_build_codebook_kernel, dim3((unsigned)n_codebooks), dim3(KVC_CB_THREADS), 0, stream, d_counts,
                       tree_format, kvc_cb_tree_nodes(tree_format), d_encode_tables, d_decode_trees, d_meta);
    return kvc_check_hip(hipGetLastError(), "kvc_build_codebook_kernel launch");
}
