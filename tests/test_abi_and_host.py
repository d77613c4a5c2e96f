"""CPU-side checks of the product: the C-ABI library loads and exports every symbol that
include/kvcomp_hip.h declares, its host-only entry points (buffer sizes, Huffman codebook) agree with the
oracle byte for byte, errors are returned instead of aborting, and the host bookkeeping mirrors
utils/compute.py.  No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import ref as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "kvcomp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from kvcomp_amd import _lib
    names = _declared()
    assert len(names) >= 15
    raw = C.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libkvcomp_hip.so does not export %s" % n
    assert sorted(_lib.EXPORTED_SYMBOLS) == names          # the Python binding covers the whole header
    assert _lib.lib().kvc_abi_version() == 2


def test_every_tuning_option_is_documented_in_the_header_and_known_to_the_library():
    """The option names listed in include/kvcomp_hip.h are exactly the ones kvc_get_option answers for (names are read
    from the header's comment and from the library's option table in csrc/kvc_host.hip)."""
    import ctypes as C
    import re
    from kvcomp_amd import _lib
    header = open(os.path.join(ROOT, "include", "kvcomp_hip.h")).read()
    block = header[header.index("Tuning knobs"):header.index("int kvc_set_option")]
    documented = set(re.findall(r'"([a-z_0-9]+)"', block))
    table = open(os.path.join(ROOT, "kvcomp_amd", "csrc", "kvc_host.hip")).read()
    known = set(re.findall(r'\{"([a-z_0-9]+)", "KVCOMP_[A-Z_0-9]+",', table))
    assert known and documented == known, (sorted(documented - known), sorted(known - documented))
    L = _lib.lib()
    for name in known:
        v = C.c_int(0)
        assert L.kvc_get_option(name.encode(), C.byref(v)) == 0, name
    assert L.kvc_get_option(b"no_such_option", C.byref(C.c_int(0))) != 0


def test_missing_library_fails_loudly(monkeypatch):
    from kvcomp_amd import _lib
    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libkvcomp_hip.so")
    with pytest.raises(_lib.KvcompError):
        _lib.lib()


def test_the_reference_module_name_resolves_to_this_library():
    """`import kvcomp_cuda` (kvcomp_cuda_extension/kvcomp_cuda.pyi): four constants and nine functions."""
    import kvcomp_cuda
    from kvcomp_amd import kvcomp_cuda as impl
    assert (kvcomp_cuda.K_VEC_LEN, kvcomp_cuda.K_VEC_PER_BLK, kvcomp_cuda.V_VEC_LEN, kvcomp_cuda.V_VEC_PER_BLK) == (128, 64, 128, 64)
    for name in ("build_codebook", "calculate_buffer_size", "k_entropy_encode_cuda_export", "v_entropy_encode_cuda_export",
                 "k_entropy_decode_cuda_export", "v_entropy_decode_cuda_export", "k_decode_and_mat_vec_mul_cuda_export",
                 "v_decode_and_mat_vec_mul_cuda_export", "k_mat_vec_mul_cuda_export"):
        assert getattr(kvcomp_cuda, name) is getattr(impl, name), name
    x = torch.zeros(2, 128, 2, 2, 64, dtype=torch.uint8)
    assert kvcomp_cuda.calculate_buffer_size(x, False, 2, 64) == impl.calculate_buffer_size(x, False, 2, 64)


def test_calculate_buffer_size_matches_reference_formula():
    """src/kernels.cu:893-917."""
    import kvcomp_amd.kvcomp_cuda as m
    t = torch.empty(16, 64, 1, 32, 128, dtype=torch.uint8)
    assert m.calculate_buffer_size(t, True, 32, 128) == (16 * 32 * 8, 16 * 64 * 32 * 2, 8, t.numel())
    t = torch.empty(8, 128, 1, 32, 128, dtype=torch.uint8)
    assert m.calculate_buffer_size(t, False, 32, 128) == (8 * 64 * 8, 8 * 64 * 64 * 2, 8, t.numel())
    with pytest.raises(RuntimeError):
        m.calculate_buffer_size(torch.empty(1, 60, 1, 1, 128, dtype=torch.uint8), True, 1, 128)
    with pytest.raises(RuntimeError):
        m.calculate_buffer_size(torch.empty(1, 64, 1, 1, 128, dtype=torch.uint8), False, 1, 128)
    assert (m.K_VEC_LEN, m.K_VEC_PER_BLK, m.V_VEC_LEN, m.V_VEC_PER_BLK) == (128, 64, 128, 64)   # export_kvcomp.cpp:9-12


def _hist_cases():
    rng = np.random.default_rng(12)
    for _ in range(120):
        k = int(rng.integers(2, 64))
        cnts = rng.integers(0, 4, size=k)
        cnts[rng.integers(0, k)] += 1
        if (cnts > 0).sum() >= 2:
            c = np.zeros(256, np.int64)
            c[:k] = cnts
            yield c
    for _ in range(40):
        syms = np.clip(np.rint(rng.standard_normal(5000) * rng.uniform(1, 6) + 20), 0, 120).astype(np.uint8)
        yield np.bincount(syms, minlength=256).astype(np.int64)


def test_host_codebook_bytes_equal_oracle_and_reference():
    import kvcomp_amd.kvcomp_cuda as m
    for counts in _hist_cases():
        shift, enc, dec = m.build_codebook_from_counts(torch.from_numpy(counts))
        code, length = O.huffman_build(counts)
        o_shift, o_enc = O.encode_table(code, length, counts)
        st, o_dec = O.decode_tree(code, length, counts)
        assert st == 0 and shift == o_shift
        assert np.array_equal(enc.numpy(), o_enc) and np.array_equal(dec.numpy(), o_dec)
        if R.available():
            syms = np.repeat(np.arange(256), counts).astype(np.uint8)
            r = R.build_codebook(syms)
            assert r[0] == shift and np.array_equal(r[1], enc.numpy()) and np.array_equal(r[2], dec.numpy())


def test_host_codebook_wide_tree_and_errors():
    import kvcomp_amd.kvcomp_cuda as m
    counts = np.zeros(256, np.int64)
    counts[:200] = np.arange(1, 201)
    with pytest.raises(RuntimeError):                       # 200 symbols do not fit the int8 tree
        m.build_codebook_from_counts(torch.from_numpy(counts))
    shift, enc, dec = m.build_codebook_from_counts(torch.from_numpy(counts), tree_format=m.TREE_I16)
    assert shift == 0 and enc.numel() == 200 * 8 and dec.numel() == (2 * 200 - 2) * 5
    code, length = O.huffman_build(counts)
    assert np.array_equal(enc.numpy(), O.encode_table(code, length, counts)[1])
    # the wide tree is the same tree as the oracle's, with int16 slots
    nodes = dec.numpy().reshape(-1, 5)
    for s in range(200):
        idx = -1
        for i in range(int(length[s])):
            bit = (int(code[s]) >> (int(length[s]) - 1 - i)) & 1
            idx = bit if idx == -1 else int(nodes[idx, 1 + 2 * bit:3 + 2 * bit].copy().view(np.int16)[0])
        assert nodes[idx, 0] == 1 and int(nodes[idx, 1:3].copy().view(np.int16)[0]) == s
    lone = np.zeros(256, np.int64)
    lone[7] = 10
    with pytest.raises(RuntimeError):
        m.build_codebook_from_counts(torch.from_numpy(lone))


def test_tail_bookkeeping_mirrors_reference():
    """utils/compute.py:59-72 and the append-one-token scenario of accuracy/reproduce_cuda_error.py:25-46."""
    from kvcomp_amd import compute as cp
    for recent in (128, 256):
        buf, total, compressed = None, 0, 0
        new = torch.arange(952).view(-1, 1, 1, 1).float()
        to_c, buf = cp.cut_tensor_ctx_len_0(buf, new, 128, recent)
        total += 952
        compressed += 0 if to_c is None else to_c.shape[0]
        for i in range(952, 952 + 300):
            to_c, buf = cp.cut_tensor_ctx_len_0(buf, torch.full((1, 1, 1, 1), float(i)), 128, recent)
            total += 1
            if to_c is not None:
                assert to_c.shape[0] % 128 == 0 and float(to_c[0, 0, 0, 0]) == compressed
                compressed += to_c.shape[0]
            assert compressed + buf.shape[0] == total
            assert buf.shape[0] < recent and (total < recent or buf.shape[0] >= recent - 128)
            assert O.blocks_to_compress(buf.shape[0], 128, recent) <= 0
    assert cp.dims_to_mask([1, 2, 3, 4]) == 0xF and cp.dims_to_mask([2, 3, 4]) == 0xE and cp.dims_to_mask([1]) == 0x1
    assert cp.QUANT_DIM["ChannelQuant"] == [3] and cp.QUANT_DIM["TokenQuant"] == [1, 4]     # utils/compute.py:138-143
