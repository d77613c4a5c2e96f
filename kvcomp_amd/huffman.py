"""utils/huffman.py of the reference -- `huffman_encode(tensor) -> (bool bitstream, {symbol: '01..'})` -- with the
histogram, the bit counting and the bitstream itself produced on the GPU (libkvcomp_hip's kvc_h2_* entry points).

The reference version is pure Python (one list append per bit, minutes per MiB); its callers only take the length
of the stream to estimate compression ratios (accuracy/cr_estimate.py:46-58).  Same results: the code is built by
the same min-heap-on-frequency construction, a lone symbol gets '0', an empty input gives an empty stream and an
empty codebook, bits follow the flattened (row-major) element order.

Limits: values must be integers (any integer or floating dtype holding integers) spanning at most 256 distinct
consecutive values, i.e. max - min <= 255 -- quantized symbols always do.
"""
import ctypes as C
from typing import Dict, Tuple

import torch

from . import _lib
from ._lib import KvcompError, check


def _symbols_u8(t: torch.Tensor):
    flat = t.reshape(-1)
    lo, hi = flat.min(), flat.max()
    lo_i, hi_i = int(lo.item()), int(hi.item())
    if hi_i - lo_i > 255:
        raise KvcompError("huffman_encode: values span %d..%d, more than 256 symbols" % (lo_i, hi_i))
    sym = (flat - lo).to(torch.uint8)
    if not torch.equal(sym.to(flat.dtype) + lo, flat):
        raise KvcompError("huffman_encode: values must be integers")
    return sym.contiguous(), lo_i


def huffman_bit_count(tensor: torch.Tensor) -> int:
    """len(huffman_encode(tensor)[0]) without materialising the stream."""
    return _encode(tensor, emit=False)[0]


def huffman_encode(tensor: torch.Tensor) -> Tuple[torch.Tensor, Dict]:
    """utils/huffman.py:15-95.  Returns (bool tensor with one element per bit, on the input's device;
    codebook {symbol: bit string}) -- symbols keyed the way `tensor.tolist()` spells them."""
    total, bits, book = _encode(tensor, emit=True)
    return bits, book


def _encode(tensor: torch.Tensor, emit: bool):
    if tensor.numel() == 0:
        return 0, torch.zeros(0, dtype=torch.bool, device=tensor.device), {}
    if not tensor.is_cuda:
        raise KvcompError("huffman_encode expects a device tensor")
    L = _lib.lib()
    sym, lo = _symbols_u8(tensor)
    n = sym.numel()
    stream = C.c_void_p(torch.cuda.current_stream(sym.device).cuda_stream)
    with torch.cuda.device(sym.device):
        counts = torch.zeros(256, dtype=torch.int64, device=sym.device)
        check(L.kvc_histogram(C.c_void_p(sym.data_ptr()), n, C.c_void_p(counts.data_ptr()), stream))
        h_counts = counts.cpu()
        code = (C.c_uint32 * 256)()
        length = (C.c_uint32 * 256)()
        check(L.kvc_h2_codes(C.cast(h_counts.data_ptr(), C.POINTER(C.c_int64)), code, length))
        scratch = torch.empty(int(L.kvc_h2_scratch_bytes(n)), dtype=torch.uint8, device=sym.device)
        total = C.c_int64(0)
        # the stream length is known from the histogram alone
        nbits = sum(int(h_counts[s]) * int(length[s]) for s in range(256))
        bits = torch.empty(nbits if emit else 0, dtype=torch.bool, device=sym.device)
        check(L.kvc_h2_encode(C.c_void_p(sym.data_ptr()), n, code, length,
                              C.c_void_p(bits.data_ptr()) if emit else None, nbits, C.c_void_p(scratch.data_ptr()),
                              scratch.numel(), C.byref(total), stream))
        assert total.value == nbits
    is_float = tensor.dtype.is_floating_point
    book = {}
    for s in range(256):
        if h_counts[s] > 0:
            key = float(s + lo) if is_float else int(s + lo)
            book[key] = format(code[s], "b").zfill(length[s]) if length[s] else ""
    return nbits, bits, book
