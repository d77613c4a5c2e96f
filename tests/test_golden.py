"""Golden vectors written by the reference's own host C++ (tests/golden/make_ref_vectors.py ran
src/huffman.cpp and src/compute.cpp through oracle/_ref): the oracle must reproduce them, and so must the
product (host codebook builder on the CPU, quantizer and bookkeeping on the GPU).  The vectors are plain
arrays, so these checks also run where no reference checkout exists."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"), allow_pickle=False)
N_CB = sum(1 for k in GOLD.files if k.startswith("cb_symbols_"))
N_Q = sum(1 for k in GOLD.files if k.startswith("q_x_"))
DIMS_TO_MASK = {(1, 2, 3, 4): O.MASK_K_BLOCK, (2, 3, 4): O.MASK_V_TOKEN, (1,): O.MASK_CHANNEL, (3, 4): O.MASK_SIM_TOKEN,
                (4,): O.MASK_VECTOR, (1, 3, 4): O.MASK_SIM_BLOCK}


def test_fixture_is_complete():
    assert N_CB >= 19 and N_Q >= 24 and len(GOLD["cut_rows"]) == len(GOLD["cut_args"]) >= 100


@pytest.mark.parametrize("i", range(N_CB))
def test_oracle_codebook_equals_reference_bytes(i):
    syms = GOLD["cb_symbols_%d" % i]
    shift, enc, dec = O.build_codebook(syms)
    assert shift == int(GOLD["cb_shift_%d" % i])
    assert np.array_equal(enc, GOLD["cb_enc_%d" % i])
    assert np.array_equal(dec, GOLD["cb_dec_%d" % i])


@pytest.mark.parametrize("i", range(N_CB))
def test_product_host_codebook_equals_reference_bytes(i):
    import kvcomp_amd.kvcomp_cuda as m
    syms = GOLD["cb_symbols_%d" % i]
    counts = torch.from_numpy(np.bincount(syms, minlength=256).astype(np.int64))
    shift, enc, dec = m.build_codebook_from_counts(counts)
    assert shift == int(GOLD["cb_shift_%d" % i])
    assert np.array_equal(enc.numpy(), GOLD["cb_enc_%d" % i])
    assert np.array_equal(dec.numpy(), GOLD["cb_dec_%d" % i])


@pytest.mark.parametrize("i", range(N_Q))
def test_oracle_quant_equals_reference_bits(i):
    x = GOLD["q_x_%d" % i].view(np.float16)
    mask = DIMS_TO_MASK[tuple(int(d) for d in GOLD["q_dims_%d" % i])]
    s16, m16, c16, _, _ = O.quant(x, mask, float(GOLD["q_eb_%d" % i]))
    assert np.array_equal(s16.view(np.uint16).ravel(), GOLD["q_sym_%d" % i].ravel())
    assert np.array_equal(m16.view(np.uint16).ravel(), GOLD["q_min_%d" % i].ravel())
    assert np.array_equal(c16.view(np.uint16).ravel(), GOLD["q_scale_%d" % i].ravel())


def test_oracle_and_product_cut_rows_equal_reference():
    from kvcomp_amd import compute
    for (buf, new, bs, recent), rows in zip(GOLD["cut_args"], GOLD["cut_rows"]):
        n = O.blocks_to_compress(int(buf + new), int(bs), int(recent))
        assert max(0, n) * bs == rows
        assert max(0, compute.blocks_to_compress(int(buf + new), int(bs), int(recent))) * bs == rows


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(N_Q))
def test_gpu_quant_equals_reference_bits(i):
    """The reference's symbols / minima as fp16 values, cast the way its caller casts them
    (models/cache/kvcomp_encode.py:97-98), against the one-kernel quantizer."""
    from kvcomp_amd import compute
    x = torch.from_numpy(GOLD["q_x_%d" % i].view(np.float16).copy()).cuda()
    dims = [int(d) for d in GOLD["q_dims_%d" % i]]
    sym, mn, sc = compute.quant(x, dims, float(GOLD["q_eb_%d" % i]))
    ref_sym = GOLD["q_sym_%d" % i].view(np.float16).astype(np.float32)
    ref_min = GOLD["q_min_%d" % i].view(np.float16).astype(np.float32)
    if np.isfinite(ref_sym).all() and ref_sym.min() >= 0 and ref_sym.max() <= 255 and np.abs(ref_min).max() <= 127:
        assert np.array_equal(sym.cpu().numpy().ravel(), ref_sym.astype(np.uint8).ravel())
        assert np.array_equal(mn.cpu().numpy().ravel(), ref_min.astype(np.int8).ravel())
    assert np.array_equal(sc.cpu().numpy().view(np.uint16).ravel(), GOLD["q_scale_%d" % i].ravel())


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(N_CB))
def test_gpu_codebook_from_device_symbols_equals_reference_bytes(i):
    """build_codebook on device symbols: GPU histogram + host heap (src/huffman.cpp:99-157)."""
    import kvcomp_amd.kvcomp_cuda as m
    syms = torch.from_numpy(GOLD["cb_symbols_%d" % i].copy()).cuda()
    shift, enc, dec = m.build_codebook([syms])
    assert shift == int(GOLD["cb_shift_%d" % i])
    assert np.array_equal(enc.cpu().numpy(), GOLD["cb_enc_%d" % i])
    assert np.array_equal(dec.cpu().numpy(), GOLD["cb_dec_%d" % i])
