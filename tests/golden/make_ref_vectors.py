#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors.npz: inputs and outputs of the REFERENCE's own host C++ for this path,
executed through oracle/_ref/libkvc_ref.so (the reference's src/huffman.cpp and src/compute.cpp compiled
where they lie by oracle/build_oracle.py).

    python tests/golden/make_ref_vectors.py        # needs the reference checkout, i.e. a built oracle/_ref

The file holds data only (numpy arrays, loaded with allow_pickle=False):

  cb_symbols_<i>, cb_shift_<i>, cb_enc_<i>, cb_dec_<i>
      build_codebook (src/huffman.cpp:99-157) on seeded symbol arrays: tie-heavy small alphabets, quantized
      Gaussians like a V cache, Laplace with outliers like the long-context stress case, all-equal counts
  q_x_<i>, q_dims_<i>, q_eb_<i>, q_sym_<i>, q_min_<i>, q_scale_<i>
      quant (src/compute.cpp:40-58) on seeded fp16 tensors [NB, BS, B, H, D] for the reduction-dimension
      lists the callers use (models/cache/kvcomp_encode.py:10-13, utils/compute.py:138-143); fp16 bit patterns
  cut_args, cut_rows
      rows cut_tensor (src/compute.cpp:13-38) hands to the compressor for (buffer_len, new_len, block, recent)

The vectors travel to machines that have no reference checkout; tests/test_golden.py checks the oracle
and the GPU path against them.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import ref as R  # noqa: E402


def codebook_inputs():
    rng = np.random.default_rng(20240611)
    out = []
    for k, hi in ((2, 3), (3, 2), (5, 2), (8, 3), (13, 2), (31, 2), (64, 2)):       # many equal counts
        cnts = rng.integers(1, hi + 1, size=k)
        out.append(rng.permutation(np.repeat(np.arange(k), cnts)).astype(np.uint8))
    for sigma in (0.8, 1.7, 3.1, 6.0):                                               # quantized Gaussian
        out.append(np.clip(np.rint(rng.standard_normal(4096) * sigma + 16), 0, 63).astype(np.uint8))
    for scale in (1.0, 2.5):                                                         # Laplace + outliers
        u = rng.random(4096) - 0.5
        x = -np.sign(u) * np.log1p(-2 * np.abs(u)) * scale
        x = np.where(rng.random(4096) < 0.02, x * 12, x)
        out.append(np.clip(np.rint(x + 30), 0, 63).astype(np.uint8))
    for k in (2, 4, 7, 16, 64):                                                      # all-equal counts
        out.append(np.repeat(np.arange(k), 3).astype(np.uint8))
    out.append(np.array([5, 5, 5, 9, 9, 63, 0, 0, 0, 0, 17], np.uint8))              # sparse alphabet
    return out


def quant_inputs():
    rng = np.random.default_rng(77)
    cases = []
    for dims, shape in (((1, 2, 3, 4), (2, 64, 1, 2, 16)),      # K block      (kvcomp_encode.py:10-13)
                        ((2, 3, 4), (1, 64, 1, 2, 16)),          # V token
                        ((1,), (2, 64, 1, 2, 16)),               # per channel  (utils/compute.py:140)
                        ((3, 4), (1, 64, 2, 2, 16)),             # token quant of the simulated path (:141)
                        ((4,), (1, 64, 2, 2, 16)),               # vector quant (:142)
                        ((1, 3, 4), (2, 64, 2, 2, 16))):         # block quant of the simulated path (:139)
        for eb in (0.05, 0.1, 0.2, 0.3):
            x = rng.standard_normal(shape).astype(np.float32)
            x *= np.exp(0.5 * rng.standard_normal(shape[-1])).astype(np.float32)
            if eb == 0.3:
                x = np.where(rng.random(shape) < 0.02, x * 50, x)
            cases.append((x.astype(np.float16), np.array(dims, np.int64), np.float32(eb)))
    return cases


def main():
    if not R.available():
        sys.exit("oracle/_ref/libkvc_ref.so is missing: run python oracle/build_oracle.py where the reference is mounted")
    data = {}
    for i, syms in enumerate(codebook_inputs()):
        shift, enc, dec = R.build_codebook(syms)
        data["cb_symbols_%d" % i] = syms
        data["cb_shift_%d" % i] = np.int64(shift)
        data["cb_enc_%d" % i] = enc
        data["cb_dec_%d" % i] = dec
    for i, (x, dims, eb) in enumerate(quant_inputs()):
        sym, mn, sc = R.quant(x, tuple(int(d) for d in dims), float(eb))
        data["q_x_%d" % i] = x.view(np.uint16)
        data["q_dims_%d" % i] = dims
        data["q_eb_%d" % i] = eb
        data["q_sym_%d" % i] = sym.view(np.uint16)
        data["q_min_%d" % i] = mn.view(np.uint16)
        data["q_scale_%d" % i] = sc.view(np.uint16)
    args, rows = [], []
    for bs in (64, 128):
        for recent in (bs, 2 * bs, 4 * bs):
            for buf in (0, 1, bs - 1, bs, 3 * bs + 5):
                for new in (1, 7, bs, 952, 4 * bs + 3):
                    args.append((buf, new, bs, recent))
                    rows.append(R.cut_rows(buf, new, bs, recent))
    data["cut_args"] = np.array(args, np.int64)
    data["cut_rows"] = np.array(rows, np.int64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_vectors.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes;", len(data), "arrays")


if __name__ == "__main__":
    main()
