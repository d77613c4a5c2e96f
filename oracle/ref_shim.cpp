// ref_shim.cpp -- flat C entry points around the REFERENCE's own host C++ (huffman.cpp, compute.cpp),
// which oracle/build_oracle.py compiles in place from the reference checkout into oracle/_ref/.
// TEST INFRASTRUCTURE ONLY: used to validate oracle/kvc_oracle.c (and to write golden vectors); the
// shipped library never sees it.  Nothing of the reference is copied here -- this file only calls the
// functions its headers declare (include/huffman.h, include/compute.h).
#include <cstring>
#include <huffman.h>
#include <compute.h>

extern "C" {

// build_codebook (src/huffman.cpp:99-157) on one uint8 tensor.
// Returns 0, or -1 if an output buffer is too small.
int kvr_build_codebook(const uint8_t *sym, int64_t n, int *shift,
                       uint8_t *enc, int64_t enc_cap, int64_t *enc_bytes,
                       uint8_t *dec, int64_t dec_cap, int64_t *dec_bytes)
{
    auto t = torch::from_blob(const_cast<uint8_t *>(sym), {n}, torch::TensorOptions().dtype(torch::kUInt8));
    auto [sh, e, d] = build_codebook({t});
    *shift = (int)sh;
    *enc_bytes = e.numel();
    *dec_bytes = d.numel();
    if (e.numel() > enc_cap || d.numel() > dec_cap) return -1;
    std::memcpy(enc, e.data_ptr(), (size_t)e.numel());
    std::memcpy(dec, d.data_ptr(), (size_t)d.numel());
    return 0;
}

// quant (src/compute.cpp:40-58) on an fp16 [NB,BS,B,H,D] tensor; dims = dimensions reduced over.
// Outputs are the three fp16 tensors it returns, flattened.
int kvr_quant(const uint16_t *x, const int64_t *shape5, const int64_t *dims, int ndims, float eb,
              uint16_t *sym_f16, uint16_t *min_f16, int64_t min_cap, uint16_t *scale_f16)
{
    auto t = torch::from_blob(const_cast<uint16_t *>(x), {shape5[0], shape5[1], shape5[2], shape5[3], shape5[4]},
                              torch::TensorOptions().dtype(torch::kHalf));
    std::vector<size_t> qd;
    for (int i = 0; i < ndims; i++) qd.push_back((size_t)dims[i]);
    auto [q, mi, sc] = quant(t, qd, eb);
    q = q.contiguous(); mi = mi.contiguous(); sc = sc.contiguous();
    if (mi.numel() > min_cap) return -1;
    std::memcpy(sym_f16, q.data_ptr(), (size_t)q.numel() * 2);
    std::memcpy(min_f16, mi.data_ptr(), (size_t)mi.numel() * 2);
    std::memcpy(scale_f16, sc.data_ptr(), (size_t)sc.numel() * 2);
    return 0;
}

// cut_tensor (src/compute.cpp:13-38): returns how many leading rows it hands to the compressor.
int64_t kvr_cut_rows(int64_t buffer_len, int64_t new_len, int64_t block_size, int64_t recent_size)
{
    auto a = torch::zeros({buffer_len, 1}, torch::kUInt8);
    auto b = torch::zeros({new_len, 1}, torch::kUInt8);
    auto [to_compress, remaining] = cut_tensor(a, b, block_size, recent_size, 0);
    return to_compress.defined() ? to_compress.size(0) : 0;
}

}  // extern "C"
