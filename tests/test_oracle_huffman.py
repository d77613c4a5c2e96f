"""Pins of the oracle's Huffman construction (H1/H2) and tables (T1/T2): the stdlib heapq driven by a
frequency-only comparison (what utils/huffman.py:13-14,46-64 runs), Kraft equality, optimal cost from an
independent merge loop, closed forms, hand-worked byte vectors, and the reference's huffman.cpp compiled into
oracle/_ref where present."""
import itertools

import numpy as np
import pytest

from oracle import oracle as O
from oracle import ref as R


def _codes_as_strings(code, length, counts):
    return {s: format(int(code[s]), "b").zfill(int(length[s])) if length[s] else "" for s in np.nonzero(counts)[0]}


def _cases():
    rng = np.random.default_rng(1)
    for k in range(2, 6):                                   # exhaustive: alphabets <= 5, counts 0..3
        for cnts in itertools.product(range(0, 4), repeat=k):
            if sum(c > 0 for c in cnts) >= 2:
                yield np.repeat(np.arange(k), cnts).astype(np.uint8)
    for _ in range(200):                                    # tie-heavy random histograms up to 200 symbols
        k = int(rng.integers(2, 200))
        cnts = rng.integers(0, 5, size=k)
        if (cnts > 0).sum() >= 2:
            yield np.repeat(np.arange(k), cnts).astype(np.uint8)
    for _ in range(60):                                     # Gaussian-shaped, like quantized KV
        yield np.clip(np.rint(rng.standard_normal(5000) * rng.uniform(1, 8) + 20), 0, 255).astype(np.uint8)
    for k in (2, 3, 7, 64, 256):                            # all-equal counts
        yield np.repeat(np.arange(k), 3).astype(np.uint8)


def test_codes_equal_stdlib_heapq_construction():
    n = 0
    for syms in _cases():
        book = O.py_huffman_codebook(syms)
        counts = np.bincount(syms, minlength=256)
        code, length = O.huffman_build(counts, h2_single=True)
        assert _codes_as_strings(code, length, counts) == book
        n += 1
    assert n > 1500


def test_kraft_prefix_free_and_optimal_cost():
    for syms in itertools.islice(_cases(), 0, None, 7):
        counts = np.bincount(syms, minlength=256).astype(np.int64)
        code, length = O.huffman_build(counts)
        present = np.nonzero(counts)[0]
        assert abs(sum(2.0 ** -int(length[s]) for s in present) - 1.0) < 1e-12            # Kraft equality
        strs = sorted(_codes_as_strings(code, length, counts).values())
        assert all(not b.startswith(a) for a, b in zip(strs, strs[1:]))                    # prefix-free
        w = sorted(int(counts[s]) for s in present)                                        # textbook cost
        cost = 0
        while len(w) > 1:
            m = w[0] + w[1]
            cost += m
            w = sorted(w[2:] + [m])
        assert cost == int(sum(int(counts[s]) * int(length[s]) for s in present))


def test_closed_forms():
    c = np.zeros(256, np.int64)
    c[5], c[9] = 3, 7                               # two symbols: first pop (smaller count) = left = '0'
    code, length = O.huffman_build(c)
    assert (int(code[5]), int(length[5]), int(code[9]), int(length[9])) == (0, 1, 1, 1)
    c[5], c[9] = 7, 7                               # tie: leaves pushed in ascending order, 5 pops first
    code, length = O.huffman_build(c)
    assert (int(code[5]), int(code[9])) == (0, 1)
    for k in (1, 2, 3, 5, 8):                       # 2^k equal counts -> every length is k
        c = np.zeros(256, np.int64)
        c[:2 ** k] = 11
        _, length = O.huffman_build(c)
        assert (length[:2 ** k] == k).all()
    c = np.zeros(256, np.int64)
    c[0], c[1], c[2] = 10, 2, 3                     # worked example: {1:'00', 2:'01', 0:'1'}
    code, length = O.huffman_build(c)
    assert [(int(code[s]), int(length[s])) for s in range(3)] == [(1, 1), (0, 2), (1, 2)]


def test_single_symbol_modes():
    c = np.zeros(256, np.int64)
    c[42] = 9
    code, length = O.huffman_build(c, h2_single=False)      # src/huffman.cpp:60-71: empty code
    assert int(length[42]) == 0
    code, length = O.huffman_build(c, h2_single=True)       # utils/huffman.py:42-44: '0'
    assert (int(code[42]), int(length[42])) == (0, 1)
    assert O.py_huffman_codebook(np.full(9, 42)) == {42: "0"}
    assert O.huffman_build(np.zeros(256, np.int64))[1].sum() == 0


def test_tables_hand_worked_bytes():
    """Codebook {0:'0', 1:'10', 2:'11'}: encode table and decode tree written out by hand from
    include/huffman.h:13-22 and the insertion rule of src/huffman.cpp:229-252."""
    counts = np.zeros(256, np.int64)
    counts[:3] = 1
    code = np.zeros(256, np.uint32)
    length = np.zeros(256, np.uint32)
    code[:3], length[:3] = [0, 2, 3], [1, 2, 2]
    shift, enc = O.encode_table(code, length, counts)
    assert shift == 0
    assert enc.tolist() == [0, 0, 0, 0, 1, 0, 0, 0, 2, 0, 0, 0, 2, 0, 0, 0, 3, 0, 0, 0, 2, 0, 0, 0]
    st, dec = O.decode_tree(code, length, counts)
    assert st == 0
    assert dec.tolist() == [1, 0, 0, 0, 2, 3, 1, 1, 1, 1, 2, 2]
    # shift: table indexed by symbol - min symbol, gaps zero filled (src/huffman.cpp:166-187)
    counts = np.zeros(256, np.int64)
    counts[[4, 6]] = 1
    code[:] = 0
    length[:] = 0
    code[[4, 6]], length[[4, 6]] = [0, 1], [1, 1]
    shift, enc = O.encode_table(code, length, counts)
    assert shift == 4 and enc.size == 24 and enc[8:16].sum() == 0 and enc[16] == 1 and enc[20] == 1


def test_tree_walk_reaches_every_symbol():
    rng = np.random.default_rng(4)
    for _ in range(50):
        syms = np.clip(np.rint(rng.standard_normal(3000) * rng.uniform(1, 6) + 15), 0, 60).astype(np.uint8)
        counts = np.bincount(syms, minlength=256).astype(np.int64)
        code, length = O.huffman_build(counts)
        st, tree = O.decode_tree(code, length, counts)
        assert st == 0 and tree.size == 3 * (2 * np.count_nonzero(counts) - 2)
        for s in np.nonzero(counts)[0]:
            idx = -1
            for i in range(int(length[s])):
                bit = (int(code[s]) >> (int(length[s]) - 1 - i)) & 1
                idx = bit if idx == -1 else int(np.int8(tree[3 * idx + 1 + bit]))
                assert idx >= 0
            assert tree[3 * idx] == 1 and tree[3 * idx + 1] == s and tree[3 * idx + 2] == s


def test_reference_int8_limits_are_flagged():
    counts = np.zeros(256, np.int64)
    counts[:70] = 5                                 # 70 symbols -> 138 nodes: child indices overflow int8
    code, length = O.huffman_build(counts)
    st, _ = O.decode_tree(code, length, counts)
    assert st == -2
    counts = np.zeros(256, np.int64)
    counts[[3, 200]] = 5                            # symbol > 127 does not fit the int8 leaf slot
    code, length = O.huffman_build(counts)
    assert O.decode_tree(code, length, counts)[0] == -2
    with pytest.raises(ValueError):
        O.build_codebook(np.array([3, 200], np.uint8))


def test_whole_tensor_bitstream_equals_string_model():
    """H2: utils/huffman.py:83-95 -- concatenated code strings of the flattened tensor, as bools."""
    rng = np.random.default_rng(6)
    for _ in range(20):
        syms = np.clip(np.rint(rng.standard_normal((7, 33)) * rng.uniform(0.5, 5) + 12), 0, 255).astype(np.uint8)
        book = O.py_huffman_codebook(syms)
        counts = np.bincount(syms.ravel(), minlength=256)
        code, length = O.huffman_build(counts, h2_single=True)
        bits = O.huffman_bits(syms, code, length)
        assert bits.dtype == bool and np.array_equal(bits, O.py_bits(syms, book))
        assert bits.size == int(sum(int(counts[s]) * int(length[s]) for s in np.nonzero(counts)[0]))


@pytest.mark.skipif(not R.available(), reason="oracle/_ref (reference C++ built in place) not present")
def test_codebook_bytes_equal_reference_cpp():
    rng = np.random.default_rng(2)
    n = 0
    for trial in range(150):
        if trial % 3 == 0:
            syms = np.clip(np.rint(rng.standard_normal(4000) * rng.uniform(1, 6) + rng.integers(0, 30)), 0, 120).astype(np.uint8)
        else:
            k = int(rng.integers(2, 60))
            cnts = rng.integers(0, 4, size=k)
            cnts[rng.integers(0, k)] += 1
            syms = np.repeat(np.arange(k), cnts).astype(np.uint8)
        if len(np.unique(syms)) < 2:
            continue
        a, b = R.build_codebook(syms), O.build_codebook(syms)
        assert a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
        n += 1
    assert n > 100
