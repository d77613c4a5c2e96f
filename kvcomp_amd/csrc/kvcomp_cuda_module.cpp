// The reference's `kvcomp_cuda` Python module as a compiled PyTorch extension over libkvcomp_hip.so.
//
// Same module name, constants and functions as kvcomp_cuda_extension/export_kvcomp.cpp:8-26 and
// kvcomp_cuda_extension/kvcomp_cuda.pyi:14-84; each function checks its tensors the way the reference's host wrappers
// do (src/kernels.cu:893-1273, src/huffman.cpp:99-157) and forwards plain pointers and sizes to the C ABI of
// include/kvcomp_hip.h on torch's current stream.  Host C++ only: no device code lives here.
//
// Deliberate differences from the reference: a failed check raises a Python RuntimeError (the reference aborts the
// process, include/utils.h:7-15); batch > 1, head_dim < 128, grouped-query heads and per-channel K scales are
// accepted; kernels run on torch's current stream instead of the legacy default stream.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <tuple>
#include <vector>

#include "kvcomp_hip.h"

namespace {

constexpr int64_t kKVecLen = 128, kKVecPerBlk = 64, kVVecLen = 128, kVVecPerBlk = 64;
constexpr int kMaskKBlock = 0xF, kMaskVToken = 0xE, kMaskChannel = 0x1, kMaskSimToken = 0xC, kMaskVector = 0x8;

void ok(int rc) { TORCH_CHECK(rc == 0, kvc_last_error()); }

void *stream_of(const torch::Tensor &t) { return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

void dev_u8(const torch::Tensor &t, const char *name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a device tensor");
    TORCH_CHECK(t.scalar_type() == torch::kUInt8, name, " must be uint8");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

template <typename T = uint8_t>
T *ptr(const torch::Tensor &t) { return (T *)t.data_ptr(); }

// [NB, BS, B, H, D] -> (tokens, bytes per token)
std::pair<int64_t, int64_t> geometry(const torch::Tensor &t5) {
    TORCH_CHECK(t5.dim() == 5, "symbol tensor must be [NB, BS, B, H, D]");
    return {t5.size(0) * t5.size(1), t5.size(2) * t5.size(3) * t5.size(4)};
}

// src/kernels.cu:893-917
std::tuple<int64_t, int64_t, int64_t, int64_t> calculate_buffer_size(const torch::Tensor &input, bool is_k, int64_t head_num,
                                                                     int64_t head_dim) {
    auto [tokens, stride] = geometry(input);
    int64_t out[4];
    ok(kvc_calculate_buffer_size(tokens, stride, is_k, head_num, head_dim, out));
    return {out[0], out[1], out[2], out[3]};
}

// src/huffman.cpp:99-157: the histogram runs on the device, the tree is built on the host
std::tuple<int64_t, torch::Tensor, torch::Tensor> build_codebook(const std::vector<torch::Tensor> &input_tensors) {
    TORCH_CHECK(!input_tensors.empty(), "input_tensors must not be empty");
    const auto dev = input_tensors[0].device();
    for (const auto &t : input_tensors) {
        TORCH_CHECK(t.device() == dev, "All input tensors must be on the same device.");
        TORCH_CHECK(t.scalar_type() == torch::kUInt8, "Input tensors must be of type uint8.");
    }
    c10::DeviceGuard guard(dev);
    auto counts = torch::zeros({256}, torch::dtype(torch::kInt64).device(dev));
    for (const auto &t : input_tensors) {
        auto c = t.contiguous();
        ok(kvc_histogram(ptr(c), c.numel(), ptr<int64_t>(counts), stream_of(c)));
    }
    auto host = counts.cpu();
    auto enc = torch::zeros({256 * 8}, torch::kUInt8), dec = torch::zeros({512 * 5}, torch::kUInt8);
    int shift = 0;
    int64_t eb = 0, db = 0;
    ok(kvc_build_codebook_host(ptr<int64_t>(host), KVC_TREE_I8, &shift, ptr(enc), enc.numel(), &eb, ptr(dec), dec.numel(), &db));
    return {shift, enc.slice(0, 0, eb).clone(), dec.slice(0, 0, db).clone()};
}

using Encoded = std::tuple<torch::Tensor, torch::Tensor, torch::Tensor>;

Encoded entropy_encode(bool is_k, const torch::Tensor &input, const torch::Tensor &encode_code_book, const torch::Tensor &block_infos,
                       const torch::Tensor &thread_infos, const torch::Tensor &idx_offset, const torch::Tensor &encoded_data,
                       int64_t base_global_offset, int64_t head_num, int64_t head_dim) {
    dev_u8(input, "input");
    dev_u8(encode_code_book, "encode_code_book");
    dev_u8(block_infos, "block_infos");
    dev_u8(thread_infos, "thread_infos");
    dev_u8(idx_offset, "idx_offset");
    dev_u8(encoded_data, "encoded_data");
    auto [tokens, stride] = geometry(input);
    int64_t sizes[4];
    ok(kvc_calculate_buffer_size(tokens, stride, is_k, head_num, head_dim, sizes));
    TORCH_CHECK(block_infos.numel() >= sizes[0], "block_infos buffer too small");
    TORCH_CHECK(thread_infos.numel() >= sizes[1], "thread_infos buffer too small");
    TORCH_CHECK(idx_offset.numel() >= sizes[2], "idx_offset buffer too small");
    c10::DeviceGuard guard(input.device());
    int64_t total = 0, max_tile = 0, max_stream = 0;
    auto fn = is_k ? kvc_k_entropy_encode : kvc_v_entropy_encode;
    ok(fn(ptr(input), tokens, stride, ptr(encode_code_book), encode_code_book.numel(), ptr(block_infos), ptr(thread_infos),
          ptr(idx_offset), ptr(encoded_data), encoded_data.numel(), (uint32_t)base_global_offset, head_num, head_dim, &total,
          &max_tile, &max_stream, stream_of(input)));
    return {encoded_data.slice(0, 0, total), block_infos.slice(0, 0, sizes[0]), thread_infos.slice(0, 0, sizes[1])};
}

// src/kernels.cu:919-966
Encoded k_entropy_encode_cuda_export(const torch::Tensor &input, const torch::Tensor &encode_code_book, const torch::Tensor &block_infos,
                                     const torch::Tensor &thread_infos, const torch::Tensor &idx_offset,
                                     const torch::Tensor &encoded_data, int64_t base_global_offset, int64_t head_num, int64_t head_dim) {
    return entropy_encode(true, input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data, base_global_offset,
                          head_num, head_dim);
}

// src/kernels.cu:968-1011
Encoded v_entropy_encode_cuda_export(const torch::Tensor &input, const torch::Tensor &encode_code_book, const torch::Tensor &block_infos,
                                     const torch::Tensor &thread_infos, const torch::Tensor &idx_offset,
                                     const torch::Tensor &encoded_data, int64_t base_global_offset, int64_t head_num, int64_t head_dim) {
    return entropy_encode(false, input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data, base_global_offset,
                          head_num, head_dim);
}

double entropy_decode(bool is_k, const torch::Tensor &in, const torch::Tensor &block_infos, const torch::Tensor &thread_infos,
                      const torch::Tensor &decode_code_book, const torch::Tensor &out, int64_t head_num, int64_t head_dim) {
    dev_u8(in, "in_tensor");
    dev_u8(block_infos, "block_infos");
    dev_u8(thread_infos, "thread_infos");
    dev_u8(decode_code_book, "decode_code_book");
    dev_u8(out, "out");
    auto [tokens, stride] = geometry(out);
    c10::DeviceGuard guard(out.device());
    float ms = 0.f;
    auto fn = is_k ? kvc_k_entropy_decode : kvc_v_entropy_decode;
    ok(fn(ptr(in), in.numel(), ptr(block_infos), block_infos.numel(), ptr(thread_infos), thread_infos.numel(),
          ptr(decode_code_book), decode_code_book.numel(), KVC_TREE_I8, ptr(out), tokens, stride, head_num, head_dim, &ms,
          stream_of(out)));
    return ms;
}

// src/kernels.cu:1013-1049
double k_entropy_decode_cuda_export(const torch::Tensor &in, const torch::Tensor &block_infos, const torch::Tensor &thread_infos,
                                    const torch::Tensor &decode_code_book, const torch::Tensor &out, int64_t head_num, int64_t head_dim) {
    return entropy_decode(true, in, block_infos, thread_infos, decode_code_book, out, head_num, head_dim);
}

// src/kernels.cu:1051-1087
double v_entropy_decode_cuda_export(const torch::Tensor &in, const torch::Tensor &block_infos, const torch::Tensor &thread_infos,
                                    const torch::Tensor &decode_code_book, const torch::Tensor &out, int64_t head_num, int64_t head_dim) {
    return entropy_decode(false, in, block_infos, thread_infos, decode_code_book, out, head_num, head_dim);
}

double fused(bool is_k, const torch::Tensor &decode_code_book, const torch::Tensor &block_infos, const torch::Tensor &thread_infos,
             const torch::Tensor &encoded_data, const torch::Tensor &quant_min_ints, const torch::Tensor &quant_scales,
             const torch::Tensor &B, const torch::Tensor &C, int64_t head_num, int64_t head_dim) {
    dev_u8(decode_code_book, "decode_code_book");
    dev_u8(block_infos, "block_infos");
    dev_u8(thread_infos, "thread_infos");
    dev_u8(encoded_data, "encoded_data");
    TORCH_CHECK(quant_min_ints.is_cuda() && quant_min_ints.scalar_type() == torch::kInt8 && quant_min_ints.is_contiguous(),
                "quant_min_ints must be a contiguous device int8 tensor");
    TORCH_CHECK(quant_scales.is_cuda() && quant_scales.scalar_type() == torch::kFloat16 && quant_scales.is_contiguous(),
                "quant_scales must be a contiguous device float16 tensor");
    TORCH_CHECK(B.is_cuda() && B.scalar_type() == torch::kFloat16 && B.is_contiguous() && B.dim() == 3,
                "B must be a contiguous 3-D device float16 tensor");
    TORCH_CHECK(C.is_cuda() && C.scalar_type() == torch::kFloat16 && C.is_contiguous(), "C must be a contiguous device float16 tensor");
    const int64_t batch = B.size(0), q_heads = B.size(1), n = quant_scales.numel();
    int64_t tokens;
    int mask;
    if (is_k) {
        TORCH_CHECK(C.dim() == 3 && C.size(0) == batch && C.size(1) == q_heads, "C must be [batch, heads, ctx]");
        TORCH_CHECK(B.size(2) == head_dim, "B must be [batch, heads, head_dim]");
        tokens = C.size(2);
        const int64_t rows = tokens / kKVecPerBlk;
        if (n == rows) mask = kMaskKBlock;
        else if (n == rows * batch * head_num * head_dim) mask = kMaskChannel;
        else TORCH_CHECK(false, "quant_scales has ", n, " elements: expected one per 64-token block (", rows,
                         ") or one per (block, batch, head, channel) (", rows * batch * head_num * head_dim, ")");
    } else {
        tokens = B.size(2);
        TORCH_CHECK(C.dim() == 4 && C.size(0) * kVVecLen == tokens && C.size(1) == batch && C.size(2) == q_heads &&
                    C.size(3) == head_dim, "C must be [ctx/128, batch, heads, head_dim]");
        if (n == tokens) mask = kMaskVToken;
        else if (n == tokens * batch) mask = kMaskSimToken;
        else if (n == tokens * batch * head_num) mask = kMaskVector;
        else TORCH_CHECK(false, "quant_scales has ", n, " elements: expected one per token (", tokens,
                         "), per (token, batch) or per (token, batch, head)");
    }
    TORCH_CHECK(quant_min_ints.numel() == n, "quant_min_ints and quant_scales must have the same number of elements");
    c10::DeviceGuard guard(B.device());
    float ms = 0.f;
    auto fn = is_k ? kvc_k_decode_and_mat_vec_mul : kvc_v_decode_and_mat_vec_mul;
    ok(fn(ptr(decode_code_book), decode_code_book.numel(), KVC_TREE_I8, ptr(block_infos), block_infos.numel(), ptr(thread_infos),
          thread_infos.numel(), ptr(encoded_data), encoded_data.numel(), ptr<int8_t>(quant_min_ints), quant_scales.data_ptr(), mask,
          B.data_ptr(), C.data_ptr(), tokens, batch, head_num, q_heads, head_dim, &ms, stream_of(B)));
    return ms;
}

// src/kernels.cu:1093-1136: C[b,h,t] = sum_i dequant(K)[t,b,h,i] * B[b,h,i]
double k_decode_and_mat_vec_mul_cuda_export(const torch::Tensor &decode_code_book, const torch::Tensor &block_infos,
                                            const torch::Tensor &thread_infos, const torch::Tensor &encoded_data,
                                            const torch::Tensor &quant_min_ints, const torch::Tensor &quant_scales,
                                            const torch::Tensor &B, const torch::Tensor &C, int64_t head_num, int64_t head_dim) {
    return fused(true, decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints, quant_scales, B, C, head_num, head_dim);
}

// src/kernels.cu:1138-1180: C[g,b,h,d] = sum_{t<128} dequant(V)[128g+t,b,h,d] * B[b,h,128g+t]
double v_decode_and_mat_vec_mul_cuda_export(const torch::Tensor &decode_code_book, const torch::Tensor &block_infos,
                                            const torch::Tensor &thread_infos, const torch::Tensor &encoded_data,
                                            const torch::Tensor &quant_min_ints, const torch::Tensor &quant_scales,
                                            const torch::Tensor &B, const torch::Tensor &C, int64_t head_num, int64_t head_dim) {
    return fused(false, decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints, quant_scales, B, C, head_num, head_dim);
}

// src/kernels.cu:1221-1273: dense fp16 baseline, out[t,b,h] = sum_i k[t,b,h,i] * q[b,h,i]
double k_mat_vec_mul_cuda_export(const torch::Tensor &k, const torch::Tensor &q, const torch::Tensor &out) {
    TORCH_CHECK(k.dim() == 4 && q.dim() == 3 && out.dim() == 3, "k [ctx,B,H,D], q [B,H,D], out [ctx,B,H]");
    const int64_t ctx = k.size(0), batch = k.size(1), heads = k.size(2), dim = k.size(3);
    TORCH_CHECK(q.size(0) == batch, "Batch size of A and B must be equal");
    TORCH_CHECK(q.size(1) == heads, "Head num of A and B must be equal");
    TORCH_CHECK(q.size(2) == dim, "Head dim of A and B must be equal");
    TORCH_CHECK(out.size(0) == ctx && out.size(1) == batch && out.size(2) == heads, "out must be [ctx, batch, heads]");
    const torch::Tensor *all[3] = {&k, &q, &out};
    const char *names[3] = {"A", "B", "C"};
    for (int i = 0; i < 3; ++i) {
        TORCH_CHECK(all[i]->is_cuda(), names[i], " must be a device tensor");
        TORCH_CHECK(all[i]->scalar_type() == torch::kFloat16, names[i], " must be of type half");
        TORCH_CHECK(all[i]->is_contiguous(), names[i], " must be contiguous");
    }
    c10::DeviceGuard guard(k.device());
    float ms = 0.f;
    ok(kvc_k_mat_vec_mul(k.data_ptr(), q.data_ptr(), out.data_ptr(), ctx, batch, heads, dim, &ms, stream_of(k)));
    return ms;
}

}  // namespace

PYBIND11_MODULE(kvcomp_cuda, m) {
    m.doc() = "kvcomp_cuda operators on AMD MI355X (libkvcomp_hip.so)";
    m.attr("K_VEC_LEN") = kKVecLen;
    m.attr("K_VEC_PER_BLK") = kKVecPerBlk;
    m.attr("V_VEC_LEN") = kVVecLen;
    m.attr("V_VEC_PER_BLK") = kVVecPerBlk;
    m.def("calculate_buffer_size", &calculate_buffer_size, "Calculate buffer size");
    m.def("build_codebook", &build_codebook, "Build Huffman codebook");
    m.def("k_entropy_encode_cuda_export", &k_entropy_encode_cuda_export, "Entropy encode K symbols");
    m.def("k_entropy_decode_cuda_export", &k_entropy_decode_cuda_export, "Entropy decode K symbols");
    m.def("k_decode_and_mat_vec_mul_cuda_export", &k_decode_and_mat_vec_mul_cuda_export, "Decode K and multiply by the query");
    m.def("k_mat_vec_mul_cuda_export", &k_mat_vec_mul_cuda_export, "Dense fp16 K times query");
    m.def("v_entropy_encode_cuda_export", &v_entropy_encode_cuda_export, "Entropy encode V symbols");
    m.def("v_entropy_decode_cuda_export", &v_entropy_decode_cuda_export, "Entropy decode V symbols");
    m.def("v_decode_and_mat_vec_mul_cuda_export", &v_decode_and_mat_vec_mul_cuda_export, "Decode V and multiply by the weights");
}
