// kvc_host.hip -- host-side plumbing of libkvcomp_hip: error reporting, the per-device scratch ring,
// buffer sizing and the host Huffman codebook builder.
#include "kvc_common.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

// ---------------------------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------------------------
static thread_local std::string g_last_error;

int kvc_fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int kvc_check_hip(hipError_t e, const char *what)
{
    if (e == hipSuccess) return 0;
    return kvc_fail(-2, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

extern "C" const char *kvc_last_error(void) { return g_last_error.c_str(); }
extern "C" int kvc_abi_version(void) { return 2; }

// ---------------------------------------------------------------------------------------------------
// tuning knobs
// ---------------------------------------------------------------------------------------------------
namespace {
struct OptionDef {
    const char *name;
    const char *env;
    int fallback;
};
const OptionDef g_option_defs[KVC_OPT_COUNT] = {
    {"fused_rows", "KVCOMP_FUSED_ROWS", -1},                     // 1: per-lane rows whenever they fit; otherwise never
    {"fused_tiles_per_wave", "KVCOMP_FUSED_TILES_PER_WAVE", 0},  // 0 choose per call
    {"fused_pair_bits", "KVCOMP_FUSED_PAIR_BITS", 8},            // widest two-symbol table index; 0 = one symbol per look-up
    {"fused_double_window", "KVCOMP_FUSED_DOUBLE_WINDOW", 1},    // 64 stream bits per refill in the one-symbol loops
    {"fused_skew", "KVCOMP_FUSED_SKEW", -1},                     // skewed payload layout: -1 choose per call, 0 never, 1 always
    {"decode_pipelined", "KVCOMP_DECODE_PIPELINED", 1},          // plain decode / decode + dequantize on the fused kernels' machinery
    {"fused_rounded", "KVCOMP_FUSED_ROUNDED", 1},                // 1: round each dequantized value to fp16 before the matvec, as the reference's dequantizer does
    {"attention_tail_in_merge", "KVCOMP_ATTENTION_TAIL_IN_MERGE", 1},   // kvc_attention_decode: V's fp16 tail inside the merge kernel
    {"fused_mfma", "KVCOMP_FUSED_MFMA", -1},                     // matrix-core kernels: -1 / 1 wherever they apply, 0 never
    {"fused_builtin_dpp", "KVCOMP_FUSED_BUILTIN_DPP", 0},        // fp32-FMA kernels: the quad permute through the compiler's intrinsic, not inline assembly
    {"fused_schedule", "KVCOMP_FUSED_SCHEDULE", -1},             // matrix-core kernels: runs of tiles per wave that shorten towards the end of the launch; -1 choose per call, 0 never, r * 10000 + p * 100 + q: runs of r for the first p % of the tiles, r / 2 for the next q %
    {"encode_one_pass", "KVCOMP_ENCODE_ONE_PASS", 1},            // tile encoder: 1: one pass (a wave counts, places by a look-back over the tiles before it, and emits its tiles); 0: two passes; 2 / 3: one pass with one / two tiles per wave
    {"fused_half_table", "KVCOMP_FUSED_HALF_TABLE", 1},          // matrix-core kernels: two-byte decode table entries for codes of 6 or 7 bits (one LDS word per bank)
    {"encode_lookback_polls", "KVCOMP_ENCODE_LOOKBACK_POLLS", 1 << 18},   // one-pass encoder: looks that may find a word not ready before a wave gives up (some tenths of a second); -1: treat every call as given up
    {"fused_schedule_v", "KVCOMP_FUSED_SCHEDULE_V", -1},         // the same for V launches: -1 follow fused_schedule (default schedule: runs that cover whole heads)
    {"fused_tiles_per_wave_v", "KVCOMP_FUSED_TILES_PER_WAVE_V", -1},   // plain grid, V launches: -1 follow fused_tiles_per_wave (default: the tiles of one head or head pair)
};
std::atomic<int> g_options[KVC_OPT_COUNT];
std::once_flag g_options_once;
void init_options()
{
    for (int i = 0; i < KVC_OPT_COUNT; i++) {
        const char *e = std::getenv(g_option_defs[i].env);
        g_options[i].store(e ? std::atoi(e) : g_option_defs[i].fallback);
    }
}
}  // namespace

int kvc_option(KvcOption which)
{
    std::call_once(g_options_once, init_options);
    return g_options[which].load(std::memory_order_relaxed);
}

extern "C" int kvc_set_option(const char *name, int value)
{
    KVC_REQUIRE(name != nullptr, "option name is NULL");
    std::call_once(g_options_once, init_options);
    for (int i = 0; i < KVC_OPT_COUNT; i++) {
        if (std::strcmp(name, g_option_defs[i].name) == 0) {
            g_options[i].store(value);
            return 0;
        }
    }
    return kvc_fail(-1, "unknown option '%s'", name);
}

extern "C" int kvc_get_option(const char *name, int *value)
{
    KVC_REQUIRE(name != nullptr && value != nullptr, "NULL argument");
    std::call_once(g_options_once, init_options);
    for (int i = 0; i < KVC_OPT_COUNT; i++) {
        if (std::strcmp(name, g_option_defs[i].name) == 0) {
            *value = g_options[i].load();
            return 0;
        }
    }
    return kvc_fail(-1, "unknown option '%s'", name);
}

// ---------------------------------------------------------------------------------------------------
// per-device scratch ring: KVC_WS_SLOTS slots handed out round-robin.  A slot is reused after
// KVC_WS_SLOTS further calls, so at most that many calls may be in flight on different streams of one
// device at the same time (calls on one stream are ordered anyway).
// A call that is being recorded into a HIP graph runs again on every replay, long after the ring has come
// round: it gets a slot of a second pool whose slots are handed out once and never again (at most
// KVC_WS_CAPTURE_SLOTS recorded calls per device and process).  Both pools are allocated by the first call on
// a device, which therefore must not be a recorded one.
// ---------------------------------------------------------------------------------------------------
constexpr int KVC_WS_SLOTS = 32;
constexpr int KVC_WS_CAPTURE_SLOTS = 480;
constexpr int KVC_MAX_DEVICES = 16;
static std::mutex g_ws_mutex;
static void *g_ws_base[KVC_MAX_DEVICES] = {};
static unsigned g_ws_next[KVC_MAX_DEVICES] = {};
static unsigned g_ws_captured[KVC_MAX_DEVICES] = {};

int kvc_workspace_slot(void **slot, void *stream)
{
    int dev = 0;
    KVC_HIP(hipGetDevice(&dev));
    KVC_REQUIRE(dev >= 0 && dev < KVC_MAX_DEVICES, "device index %d out of range", dev);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (stream) KVC_HIP(hipStreamIsCapturing((hipStream_t)stream, &capturing));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (!g_ws_base[dev]) {
        KVC_REQUIRE(capturing == hipStreamCaptureStatusNone,
                    "the first call on a device allocates the library's scratch memory and cannot be recorded into a graph: "
                    "make one call outside the capture first");
        KVC_HIP(hipMalloc(&g_ws_base[dev], (size_t)(KVC_WS_SLOTS + KVC_WS_CAPTURE_SLOTS) * KVC_WS_SLOT_BYTES));
    }
    unsigned k;
    if (capturing != hipStreamCaptureStatusNone) {
        KVC_REQUIRE(g_ws_captured[dev] < (unsigned)KVC_WS_CAPTURE_SLOTS,
                    "more than %d calls that need scratch memory have been recorded into graphs on this device", KVC_WS_CAPTURE_SLOTS);
        k = KVC_WS_SLOTS + g_ws_captured[dev]++;
    } else {
        k = g_ws_next[dev]++ % KVC_WS_SLOTS;
    }
    *slot = (char *)g_ws_base[dev] + (size_t)k * KVC_WS_SLOT_BYTES;
    return 0;
}

// ---------------------------------------------------------------------------------------------------
// calculate_buffer_size (kvcomp_cuda_extension/src/kernels.cu:893-917)
// ---------------------------------------------------------------------------------------------------
extern "C" int kvc_calculate_buffer_size(int64_t tokens, int64_t stride, int is_k, int64_t head_num,
                                         int64_t head_dim, int64_t out4[4])
{
    (void)head_num;
    KVC_REQUIRE(tokens >= 0 && stride > 0, "tokens/stride must be positive");
    KVC_REQUIRE(head_dim > 0 && head_dim <= KVC_K_VEC_LEN && head_dim % 4 == 0, "head_dim must be a multiple of 4, <= 128");
    int64_t numel = tokens * stride, vec_num, tile_num;
    if (is_k) {
        KVC_REQUIRE(tokens % KVC_K_VEC_PER_BLK == 0, "Context length must be divisible by K_VEC_PER_BLK");
        KVC_REQUIRE(stride % head_dim == 0, "Hidden dim must be divisible by head_dim");
        vec_num = numel / head_dim;
        tile_num = vec_num / KVC_K_VEC_PER_BLK;
    } else {
        KVC_REQUIRE(tokens % KVC_V_VEC_LEN == 0, "Context length must be divisible by V_VEC_LEN");
        KVC_REQUIRE(stride % KVC_V_VEC_PER_BLK == 0, "Hidden dim must be divisible by V_VEC_PER_BLK");
        vec_num = numel / KVC_V_VEC_LEN;
        tile_num = vec_num / KVC_V_VEC_PER_BLK;
    }
    out4[0] = tile_num * 8;
    out4[1] = vec_num * 2;
    out4[2] = 8;
    out4[3] = numel;   // K/V_ENCODE_PREALLOCATE_RATIO = 1 (include/kernels.h:14,20)
    return 0;
}

// ---------------------------------------------------------------------------------------------------
// Host Huffman codebook (kvcomp_cuda_extension/src/huffman.cpp:34-157, 166-187, 229-252).
//
// The reference pushes one leaf per occurring symbol, in ascending symbol order, into a
// std::priority_queue that compares frequencies only, and merges the two smallest until one node is
// left (first pop = left = bit 0).  Which of several equal-frequency nodes comes out first is decided by
// the array-heap algorithm itself, so the heap is spelled out here: push appends and sifts up while the
// new key is strictly smaller than its parent; pop moves the root hole down to a leaf, always towards
// the smaller child and towards the right child on a tie, then drops the former last element into the
// hole and sifts it up.  (Python's heapq behaves identically, which is how utils/huffman.py:46-64
// arrives at the same codes.)
// ---------------------------------------------------------------------------------------------------
namespace {
struct HNode {
    int64_t f;
    int left, right, sym;
};

struct FreqHeap {
    std::vector<int> h;
    const std::vector<HNode> &nodes;
    explicit FreqHeap(const std::vector<HNode> &n) : nodes(n) {}
    bool less(int a, int b) const { return nodes[a].f < nodes[b].f; }
    void push(int x)
    {
        h.push_back(x);
        size_t pos = h.size() - 1;
        while (pos > 0) {
            size_t par = (pos - 1) >> 1;
            if (!less(x, h[par])) break;
            h[pos] = h[par];
            pos = par;
        }
        h[pos] = x;
    }
    int pop()
    {
        int last = h.back();
        h.pop_back();
        if (h.empty()) return last;
        int top = h[0];
        size_t pos = 0, child = 1, n = h.size();
        while (child < n) {
            size_t right = child + 1;
            if (right < n && !less(h[child], h[right])) child = right;
            h[pos] = h[child];
            pos = child;
            child = 2 * pos + 1;
        }
        while (pos > 0) {
            size_t par = (pos - 1) >> 1;
            if (!less(last, h[par])) break;
            h[pos] = h[par];
            pos = par;
        }
        h[pos] = last;
        return top;
    }
};
}  // namespace

// code/length per symbol; returns number of distinct symbols or -1 when a code exceeds 32 bits.
static int kvc_huffman_codes(const int64_t *counts, uint32_t code[256], uint32_t length[256])
{
    std::vector<HNode> nodes;
    nodes.reserve(512);
    FreqHeap heap(nodes);
    for (int s = 0; s < 256; s++) {
        code[s] = 0;
        length[s] = 0;
        if (counts[s] > 0) {
            nodes.push_back({counts[s], -1, -1, s});
            heap.push((int)nodes.size() - 1);
        }
    }
    int distinct = (int)nodes.size();
    if (distinct < 2) return distinct;   // 0 symbols: nothing; 1 symbol: empty code (huffman.cpp:60-71)
    while (heap.h.size() > 1) {
        int a = heap.pop();
        int b = heap.pop();
        nodes.push_back({nodes[a].f + nodes[b].f, a, b, -1});
        heap.push((int)nodes.size() - 1);
    }
    struct Item { int node; uint64_t code; int len; };
    std::vector<Item> stack{{heap.h[0], 0, 0}};
    while (!stack.empty()) {
        Item it = stack.back();
        stack.pop_back();
        const HNode &nd = nodes[it.node];
        if (nd.left < 0) {
            if (it.len > 32) return -1;
            code[nd.sym] = (uint32_t)it.code;
            length[nd.sym] = (uint32_t)it.len;
        } else {
            if (it.len >= 63) return -1;
            stack.push_back({nd.right, (it.code << 1) | 1u, it.len + 1});
            stack.push_back({nd.left, it.code << 1, it.len + 1});
        }
    }
    return distinct;
}

// The same construction with the lone-symbol rule of utils/huffman.py:42-44 (code '0', one bit).
int kvc_huffman_codes_h2(const int64_t *counts, uint32_t code[256], uint32_t length[256])
{
    const int distinct = kvc_huffman_codes(counts, code, length);
    if (distinct == 1)
        for (int s = 0; s < 256; s++)
            if (counts[s] > 0) length[s] = 1;
    return distinct;
}

extern "C" int kvc_build_codebook_host(const int64_t *h_counts256, int tree_format, int *shift,
                                       uint8_t *h_encode_table, int64_t encode_cap, int64_t *encode_bytes,
                                       uint8_t *h_decode_tree, int64_t decode_cap, int64_t *decode_bytes)
{
    KVC_REQUIRE(tree_format == KVC_TREE_I8 || tree_format == KVC_TREE_I16, "unknown tree format %d", tree_format);
    uint32_t code[256], length[256];
    int distinct = kvc_huffman_codes(h_counts256, code, length);
    KVC_REQUIRE(distinct >= 0, "a Huffman code is longer than 32 bits");
    KVC_REQUIRE(distinct >= 2, "a codebook needs at least two distinct symbols (got %d): the reference assigns a "
                               "lone symbol the empty code, which cannot be decoded", distinct);
    int mn = 255, mx = 0;
    for (int s = 0; s < 256; s++)
        if (h_counts256[s] > 0) {
            if (s < mn) mn = s;
            if (s > mx) mx = s;
        }
    *shift = mn;
    // encode table: index = symbol - min symbol, absent symbols stay zero (huffman.cpp:166-187)
    int64_t eb = (int64_t)(mx - mn + 1) * 8;
    KVC_REQUIRE(eb <= encode_cap, "encode table needs %lld bytes", (long long)eb);
    std::memset(h_encode_table, 0, (size_t)eb);
    for (int s = mn; s <= mx; s++) {
        if (h_counts256[s] <= 0) continue;
        std::memcpy(h_encode_table + (size_t)(s - mn) * 8, &code[s], 4);
        std::memcpy(h_encode_table + (size_t)(s - mn) * 8 + 4, &length[s], 4);
    }
    *encode_bytes = eb;
    // decode tree: insert symbols in ascending order, appending nodes on demand (huffman.cpp:229-252)
    struct TNode { bool leaf; int child[2]; };
    std::vector<TNode> tree(2, TNode{false, {-1, -1}});
    for (int s = 0; s < 256; s++) {
        if (h_counts256[s] <= 0) continue;
        int idx = -1, last = -1;
        for (uint32_t i = 0; i < length[s]; i++) {
            int bit = (int)((code[s] >> (length[s] - 1 - i)) & 1u);
            idx = (idx == -1) ? bit : tree[idx].child[bit];
            if (idx == -1) {
                tree.push_back(TNode{false, {-1, -1}});
                idx = (int)tree.size() - 1;
                tree[last].child[bit] = idx;
            }
            last = idx;
        }
        tree[idx].leaf = true;
        tree[idx].child[0] = tree[idx].child[1] = s;
    }
    int64_t db = (int64_t)tree.size() * tree_format;
    KVC_REQUIRE(db <= decode_cap, "decode tree needs %lld bytes", (long long)db);
    if (tree_format == KVC_TREE_I8) {
        KVC_REQUIRE(tree.size() <= 128 && mx <= 127,
                    "code not representable in the reference's int8 tree (%zu nodes, max symbol %d): "
                    "use KVC_TREE_I16", tree.size(), mx);
        for (size_t n = 0; n < tree.size(); n++) {
            h_decode_tree[3 * n] = tree[n].leaf ? 1 : 0;
            h_decode_tree[3 * n + 1] = (uint8_t)(int8_t)tree[n].child[0];
            h_decode_tree[3 * n + 2] = (uint8_t)(int8_t)tree[n].child[1];
        }
    } else {
        for (size_t n = 0; n < tree.size(); n++) {
            int16_t a = (int16_t)tree[n].child[0], b = (int16_t)tree[n].child[1];
            h_decode_tree[5 * n] = tree[n].leaf ? 1 : 0;
            std::memcpy(h_decode_tree + 5 * n + 1, &a, 2);
            std::memcpy(h_decode_tree + 5 * n + 3, &b, 2);
        }
    }
    *decode_bytes = db;
    return 0;
}
