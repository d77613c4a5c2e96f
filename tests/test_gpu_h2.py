"""The whole-tensor Huffman coder (utils/huffman.py of the reference) on the GPU against the stdlib-heapq model
of that file (oracle.py_huffman_codebook / py_bits) and, at larger sizes, the C oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cases():
    rng = np.random.default_rng(77)
    yield "two symbols", np.array([3, 3, 5, 3, 5, 3], np.int64)
    yield "lone symbol", np.full(37, 9, np.int64)
    yield "all ties over 8", np.tile(np.arange(8), 5)
    yield "ties over 5 (not a power of two)", np.tile(np.arange(10, 15), 7)
    yield "negative values", rng.integers(-7, 4, size=1500)
    yield "gaussian symbols", np.clip(np.rint(rng.normal(6, 2.0, size=(3, 5, 300))), 0, 15).astype(np.int64)
    yield "skewed", rng.choice(np.arange(12), p=np.array([2.0 ** -(i + 1) for i in range(11)] + [2.0 ** -11]), size=5000)
    yield "one past a chunk", rng.integers(0, 6, size=1025)
    yield "wide alphabet", rng.integers(0, 256, size=20000)


@pytest.mark.parametrize("name,vals", list(_cases()), ids=[c[0] for c in _cases()])
@pytest.mark.parametrize("dtype", [torch.int64, torch.uint8, torch.float16])
def test_matches_heapq_model(name, vals, dtype):
    from kvcomp_amd.huffman import huffman_bit_count, huffman_encode
    if dtype == torch.uint8 and vals.min() < 0:
        pytest.skip("negative values do not fit uint8")
    t = torch.from_numpy(np.asarray(vals)).to(dtype).to(DEV)
    bits, book = huffman_encode(t)
    ref_book = O.py_huffman_codebook(vals)
    ref_bits = O.py_bits(vals, ref_book)
    assert bits.dtype == torch.bool and bits.device.type == "cuda"
    assert {int(k): v for k, v in book.items()} == ref_book
    assert all(isinstance(k, float if dtype == torch.float16 else int) for k in book)
    assert np.array_equal(bits.cpu().numpy(), ref_bits)
    assert huffman_bit_count(t) == ref_bits.size


def test_empty_input():
    from kvcomp_amd.huffman import huffman_encode
    bits, book = huffman_encode(torch.zeros(0, dtype=torch.int64, device=DEV))
    assert bits.numel() == 0 and bits.dtype == torch.bool and book == {}


def test_rejects_what_it_cannot_code():
    from kvcomp_amd._lib import KvcompError
    from kvcomp_amd.huffman import huffman_encode
    with pytest.raises(KvcompError):
        huffman_encode(torch.tensor([0, 300], device=DEV))
    with pytest.raises(KvcompError):
        huffman_encode(torch.tensor([0.5, 1.0], device=DEV))
    with pytest.raises(KvcompError):
        huffman_encode(torch.tensor([1, 2]))


def test_large_tensor_against_c_oracle_and_round_trip():
    """4 Mi symbols of a quantized K block: bitstream equal to the C oracle's, length = sum count * len, and
    decoding the stream with the returned codebook restores the tensor."""
    from kvcomp_amd.huffman import huffman_encode
    rng = np.random.default_rng(5)
    vals = np.clip(np.rint(rng.laplace(8, 1.6, size=(64, 256, 256))), 0, 31).astype(np.uint8)
    bits, book = huffman_encode(torch.from_numpy(vals).to(DEV))
    counts = np.bincount(vals.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts, h2_single=True)
    assert bits.numel() == int((counts * length[:256]).sum())
    assert np.array_equal(bits.cpu().numpy(), O.huffman_bits(vals, code, length))
    # prefix decode of the first 100 000 bits
    inv = {v: k for k, v in book.items()}
    got, cur = [], ""
    for b in bits[:100000].cpu().numpy():
        cur += "1" if b else "0"
        if cur in inv:
            got.append(inv[cur])
            cur = ""
    assert np.array_equal(np.array(got, np.uint8), vals.ravel()[:len(got)]) and len(got) > 20000
