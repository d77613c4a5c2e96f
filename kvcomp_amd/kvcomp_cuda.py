"""Drop-in mirror of the reference's `kvcomp_cuda` operator module for AMD MI355X.

Same names, argument order and meaning as kvcomp_cuda_extension/kvcomp_cuda.pyi:14-84 and
kvcomp_cuda_extension/export_kvcomp.cpp:8-26 (4 constants + 9 functions); every call goes through the C
ABI of libkvcomp_hip.so (include/kvcomp_hip.h) on torch's current stream.  To make the reference's own
callers pick it up:

    import sys, kvcomp_amd.kvcomp_cuda as m; sys.modules["kvcomp_cuda"] = m

Differences from the reference, all deliberate:
  * failed checks raise KvcompError (a RuntimeError) instead of aborting the process
    (include/utils.h:7-15);
  * tile payloads are laid out in tile order, not in the arrival order of a global atomic
    (src/kernels.cu:472-479) -- per-tile bytes, thread_infos and byte counts are identical;
  * batch > 1, head_dim < 128 (multiples of 8), grouped-query heads (B/q has more heads than head_num)
    and per-channel K scales are accepted where the reference asserts or silently misbehaves;
  * kernels run on torch's current stream rather than the legacy default stream.
"""
import ctypes as C
from typing import List, Tuple

import torch

from . import _lib
from ._lib import KvcompError, check  # noqa: F401

# export_kvcomp.cpp:9-12
K_VEC_LEN = 128
K_VEC_PER_BLK = 64
V_VEC_LEN = 128
V_VEC_PER_BLK = 64

# largest tile payload of the most recent encode call (a sizing hint for the table-driven fused decoders)
last_encode_max_tile_bytes = 0      # largest tile payload / longest lane stream of the latest encode call:
last_encode_max_stream_bytes = 0    # sizing hints for the table-driven fused decoders

MASK_K_BLOCK, MASK_V_TOKEN, MASK_CHANNEL, MASK_SIM_TOKEN, MASK_VECTOR, MASK_SIM_BLOCK = 0xF, 0xE, 0x1, 0xC, 0x8, 0xD
TREE_I8, TREE_I16 = 3, 5


def _ptr(t: torch.Tensor):
    return C.c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require(cond, msg):
    if not cond:
        raise KvcompError(msg)


def _dev_u8(t, name):
    _require(t.is_cuda, "%s must be a device tensor" % name)
    _require(t.dtype == torch.uint8, "%s must be uint8" % name)
    _require(t.is_contiguous(), "%s must be contiguous" % name)


def _geometry(t5: torch.Tensor):
    _require(t5.dim() == 5, "symbol tensor must be [NB, BS, B, H, D]")
    tokens = t5.shape[0] * t5.shape[1]
    stride = t5.shape[2] * t5.shape[3] * t5.shape[4]
    return tokens, stride


def calculate_buffer_size(input: torch.Tensor, is_k: bool, head_num: int, head_dim: int) -> Tuple[int, int, int, int]:
    """src/kernels.cu:893-917: (block_infos, thread_infos, idx_offset, payload pre-allocation) in bytes."""
    tokens, stride = _geometry(input)
    out = (C.c_int64 * 4)()
    check(_lib.lib().kvc_calculate_buffer_size(tokens, stride, int(bool(is_k)), head_num, head_dim, out))
    return tuple(int(v) for v in out)


def build_codebook(input_tensors: List[torch.Tensor], tree_format: int = TREE_I8) -> Tuple[int, torch.Tensor, torch.Tensor]:
    """src/huffman.cpp:99-157: histogram of all inputs -> (shift, encode table, decode tree) as CPU uint8
    tensors.  The histogram runs on the device the inputs live on (one 2 KiB copy back, where the
    reference issues 256 .item() reads, huffman.cpp:42)."""
    return build_codebook_from_counts(symbol_counts(input_tensors), tree_format)


def symbol_counts(input_tensors: List[torch.Tensor]) -> torch.Tensor:
    """256-bin histogram of device uint8 tensors (torch::bincount in src/huffman.cpp:105-109), as a CPU int64 tensor."""
    _require(len(input_tensors) > 0, "input_tensors must not be empty")
    dev = input_tensors[0].device
    for t in input_tensors:
        _require(t.device == dev, "All input tensors must be on the same device.")
        _require(t.dtype == torch.uint8, "Input tensors must be of type uint8.")
    L = _lib.lib()
    with torch.cuda.device(dev):
        counts = torch.zeros(256, dtype=torch.int64, device=dev)
        for t in input_tensors:
            t = t.contiguous()
            check(L.kvc_histogram(_ptr(t), t.numel(), _ptr(counts), _stream(t)))
        return counts.cpu()


def build_codebook_from_counts(counts: torch.Tensor, tree_format: int = TREE_I8):
    """Host half of build_codebook: int64[256] counts (CPU) -> (shift, encode table, decode tree)."""
    counts = counts.to(dtype=torch.int64, device="cpu").contiguous()
    _require(counts.numel() == 256, "Counts tensor must have 256 elements.")
    enc = torch.zeros(256 * 8, dtype=torch.uint8)
    dec = torch.zeros(512 * 5, dtype=torch.uint8)
    shift = C.c_int(0)
    eb, db = C.c_int64(0), C.c_int64(0)
    check(_lib.lib().kvc_build_codebook_host(C.cast(counts.data_ptr(), C.POINTER(C.c_int64)), tree_format, C.byref(shift),
                                             _ptr(enc), enc.numel(), C.byref(eb), _ptr(dec), dec.numel(), C.byref(db)))
    return shift.value, enc[:eb.value].clone(), dec[:db.value].clone()


def symbol_counts_chunks(symbols: torch.Tensor, n_chunks: int) -> torch.Tensor:
    """One 256-bin histogram per equal chunk of a contiguous device uint8 tensor (e.g. per 64-token block), as a
    device int64 tensor [n_chunks, 256]; nothing waits for the host."""
    _dev_u8(symbols, "symbols")
    _require(symbols.is_contiguous() and n_chunks > 0 and symbols.numel() % n_chunks == 0, "symbols must split into equal chunks")
    with torch.cuda.device(symbols.device):
        counts = torch.zeros(n_chunks, 256, dtype=torch.int64, device=symbols.device)
        check(_lib.lib().kvc_histogram_chunks(_ptr(symbols), symbols.numel() // n_chunks, n_chunks, _ptr(counts), _stream(symbols)))
    return counts


def build_codebook_device(counts: torch.Tensor, tree_format: int = TREE_I8):
    """build_codebook (src/huffman.cpp:99-157) for every row of a device int64 tensor [n, 256], on the device.
    Returns device tensors (encode tables uint8 [n, 2048], decode trees uint8 [n, capacity], meta int32 [n, 4] =
    {shift, encode table bytes, decode tree bytes, status}); rows with a non-zero status hold no code (1: fewer than
    two symbols, 2: a code beyond 32 bits, 4: not representable in the int8 tree).  The trees are padded to their
    capacity, which is the `tree_bytes` to give kvc_build_lut."""
    _require(counts.is_cuda and counts.dtype == torch.int64 and counts.dim() == 2 and counts.shape[1] == 256 and
             counts.is_contiguous(), "counts must be a contiguous device int64 tensor [n, 256]")
    n = counts.shape[0]
    cap = int(_lib.lib().kvc_codebook_tree_capacity(tree_format))
    _require(cap > 0, "unknown tree format")
    with torch.cuda.device(counts.device):
        enc = torch.empty(n, 2048, dtype=torch.uint8, device=counts.device)
        trees = torch.empty(n, cap, dtype=torch.uint8, device=counts.device)
        meta = torch.empty(n, 4, dtype=torch.int32, device=counts.device)
        check(_lib.lib().kvc_build_codebook_device(_ptr(counts), n, tree_format, _ptr(enc), _ptr(trees), _ptr(meta), _stream(counts)))
    return enc, trees, meta


def _entropy_encode(is_k, input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data,
                    base_global_offset, head_num, head_dim):
    for t, n in ((input, "input"), (encode_code_book, "encode_code_book"), (block_infos, "block_infos"),
                 (thread_infos, "thread_infos"), (idx_offset, "idx_offset"), (encoded_data, "encoded_data")):
        _dev_u8(t, n)
    tokens, stride = _geometry(input)
    sizes = calculate_buffer_size(input, is_k, head_num, head_dim)
    _require(block_infos.numel() >= sizes[0], "block_infos buffer too small")
    _require(thread_infos.numel() >= sizes[1], "thread_infos buffer too small")
    _require(idx_offset.numel() >= sizes[2], "idx_offset buffer too small")
    total, max_tile, max_stream = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    fn = _lib.lib().kvc_k_entropy_encode if is_k else _lib.lib().kvc_v_entropy_encode
    with torch.cuda.device(input.device):
        check(fn(_ptr(input), tokens, stride, _ptr(encode_code_book), encode_code_book.numel(), _ptr(block_infos),
                 _ptr(thread_infos), _ptr(idx_offset), _ptr(encoded_data), encoded_data.numel(),
                 int(base_global_offset) & 0xFFFFFFFF, head_num, head_dim, C.byref(total), C.byref(max_tile), C.byref(max_stream),
                 _stream(input)))
    global last_encode_max_tile_bytes, last_encode_max_stream_bytes
    last_encode_max_tile_bytes = int(max_tile.value)
    last_encode_max_stream_bytes = int(max_stream.value)
    return encoded_data[:total.value], block_infos[:sizes[0]], thread_infos[:sizes[1]]


def buffer_sizes(tokens: int, stride: int, is_k: bool, head_num: int, head_dim: int) -> Tuple[int, int, int, int]:
    """calculate_buffer_size (src/kernels.cu:893-917) from the geometry alone."""
    out4 = (C.c_int64 * 4)()
    check(_lib.lib().kvc_calculate_buffer_size(tokens, stride, int(is_k), head_num, head_dim, out4))
    return tuple(int(v) for v in out4)


def store_fused_supported(is_k: bool, quant_mask: int, batch: int, head_num: int, head_dim: int) -> bool:
    return bool(_lib.lib().kvc_store_fused_supported(int(is_k), quant_mask, batch, head_num, head_dim))


def store_fused(is_k: bool, cache: torch.Tensor, quant_mask: int, quant_scale_rel: float, encode_code_book, min_ints, scales,
                block_infos, thread_infos, idx_offset, encoded_data, base_global_offset: int):
    """Quantize + Huffman-encode fp16 cache rows [T, B, H, D] in one library call (no counterpart in the reference,
    which runs quant and the encoder separately: models/cache/kvcomp_encode.py:86-112).  min_ints (int8) and scales
    (fp16) receive the group parameters; returns views (payload, block_infos, thread_infos) like the encoders."""
    _require(cache.is_cuda and cache.dtype == torch.float16 and cache.dim() == 4 and cache.is_contiguous(),
             "cache must be a contiguous device float16 tensor [T, B, H, D]")
    for t, n in ((encode_code_book, "encode_code_book"), (block_infos, "block_infos"), (thread_infos, "thread_infos"),
                 (idx_offset, "idx_offset"), (encoded_data, "encoded_data")):
        _dev_u8(t, n)
    T, B, H, D = cache.shape
    sizes = buffer_sizes(T, B * H * D, is_k, H, D)
    _require(block_infos.numel() >= sizes[0], "block_infos buffer too small")
    _require(thread_infos.numel() >= sizes[1], "thread_infos buffer too small")
    _require(idx_offset.numel() >= sizes[2], "idx_offset buffer too small")
    groups = _lib.lib().kvc_quant_groups(T // 64, 64, B, H, D, quant_mask)
    _require(min_ints.dtype == torch.int8 and min_ints.numel() >= groups and min_ints.is_cuda, "min_ints: int8 device tensor of the group count")
    _require(scales.dtype == torch.float16 and scales.numel() >= groups and scales.is_cuda, "scales: fp16 device tensor of the group count")
    total, max_tile, max_stream = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    with torch.cuda.device(cache.device):
        check(_lib.lib().kvc_store_fused(int(is_k), _ptr(cache), T, B, H, D, quant_mask, float(quant_scale_rel),
                                         _ptr(encode_code_book), encode_code_book.numel(), _ptr(min_ints), _ptr(scales),
                                         _ptr(block_infos), _ptr(thread_infos), _ptr(idx_offset), _ptr(encoded_data),
                                         encoded_data.numel(), int(base_global_offset) & 0xFFFFFFFF, C.byref(total),
                                         C.byref(max_tile), C.byref(max_stream), _stream(cache)))
    global last_encode_max_tile_bytes, last_encode_max_stream_bytes
    last_encode_max_tile_bytes = int(max_tile.value)
    last_encode_max_stream_bytes = int(max_stream.value)
    return encoded_data[:total.value], block_infos[:sizes[0]], thread_infos[:sizes[1]]


def encode_async(is_k: bool, *, batch: int, head_num: int, head_dim: int, tokens: int, encode_tables: torch.Tensor,
                 table_bytes: int, block_infos: torch.Tensor, thread_infos: torch.Tensor, encoded: torch.Tensor,
                 symbols: torch.Tensor = None, cache: torch.Tensor = None, quant_mask: int = 0, eb: float = 0.0,
                 min_ints: torch.Tensor = None, scales: torch.Tensor = None, table_stride: int = 0, rows_per_codebook: int = 0,
                 codebook_meta: torch.Tensor = None, base_global_offset: int = 0, stream_bytes: torch.Tensor = None,
                 result: torch.Tensor = None):
    """kvc_encode_async: queue one encode (from `symbols`, or quantizing `cache` on the fly into min_ints / scales) with
    one table per `rows_per_codebook` tile rows, and return without waiting.  `result` (device int32[8], zeroed once)
    and `stream_bytes` (device int32[1]: payload bytes already in `encoded`, moved on by the call) stay on the device;
    encode_result() reads them.  The output tensors are written from their first element on."""
    job = _lib.EncodeJob()
    job.is_k, job.quant_mask, job.eb = int(is_k), int(quant_mask), float(eb)
    _require((symbols is None) != (cache is None), "give either symbols or cache")
    dev = (symbols if symbols is not None else cache).device
    if symbols is not None:
        _dev_u8(symbols, "symbols")
        _require(symbols.is_contiguous() and symbols.numel() == tokens * batch * head_num * head_dim, "symbols: wrong size")
        job.d_sym = symbols.data_ptr()
    else:
        _require(cache.is_cuda and cache.dtype == torch.float16 and cache.is_contiguous() and
                 cache.numel() == tokens * batch * head_num * head_dim, "cache must be a contiguous device float16 tensor [T, B, H, D]")
        groups = _lib.lib().kvc_quant_groups(tokens // 64, 64, batch, head_num, head_dim, quant_mask)
        _require(min_ints is not None and min_ints.dtype == torch.int8 and min_ints.numel() >= groups and min_ints.is_cuda,
                 "min_ints: int8 device tensor of the group count")
        _require(scales is not None and scales.dtype == torch.float16 and scales.numel() >= groups and scales.is_cuda,
                 "scales: fp16 device tensor of the group count")
        job.d_x_f16, job.d_min_i8, job.d_scale_f16 = cache.data_ptr(), min_ints.data_ptr(), scales.data_ptr()
    sizes = buffer_sizes(tokens, batch * head_num * head_dim, is_k, head_num, head_dim)
    for t, n, need in ((encode_tables, "encode_tables", table_bytes), (block_infos, "block_infos", sizes[0]),
                       (thread_infos, "thread_infos", sizes[1]), (encoded, "encoded", 0)):
        _dev_u8(t, n)
        _require(t.numel() >= need, n + " buffer too small")
    job.tokens, job.batch, job.heads, job.head_dim = tokens, batch, head_num, head_dim
    job.d_encode_tables, job.encode_table_bytes = encode_tables.data_ptr(), table_bytes
    job.table_stride_bytes, job.rows_per_codebook = table_stride, rows_per_codebook
    if rows_per_codebook:
        rows = tokens // (K_VEC_PER_BLK if is_k else V_VEC_LEN)
        n_books = -(-rows // rows_per_codebook)
        _require(encode_tables.numel() >= (n_books - 1) * table_stride + table_bytes, "encode_tables holds too few tables")
        if codebook_meta is not None:
            _require(codebook_meta.is_cuda and codebook_meta.dtype == torch.int32 and codebook_meta.numel() >= 4 * n_books,
                     "codebook_meta: device int32 [n, 4]")
    if codebook_meta is not None:
        job.d_codebook_meta = codebook_meta.data_ptr()
    job.d_block_infos, job.d_thread_infos = block_infos.data_ptr(), thread_infos.data_ptr()
    job.d_encoded, job.encoded_cap = encoded.data_ptr(), encoded.numel()
    job.base_global_offset = int(base_global_offset) & 0xFFFFFFFF
    for t, n in ((stream_bytes, "stream_bytes"), (result, "result")):
        if t is not None:
            _require(t.is_cuda and t.dtype == torch.int32 and t.is_contiguous(), n + ": device int32 tensor")
    _require(result is None or result.numel() >= 8, "result: 8 words")
    if stream_bytes is not None:
        job.d_stream_bytes = stream_bytes.data_ptr()
    if result is not None:
        job.d_result = result.data_ptr()
    with torch.cuda.device(dev):
        check(_lib.lib().kvc_encode_async(C.byref(job), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))


def encode_result(result: torch.Tensor, encoded_cap: int):
    """kvc_encode_result: wait for the stream, raise if any call sharing `result` failed, and return
    (payload bytes of the latest call, largest tile payload, longest lane stream, tiles encoded so far)."""
    total, max_tile, max_stream, tiles = C.c_int64(0), C.c_int64(0), C.c_int64(0), C.c_int64(0)
    with torch.cuda.device(result.device):
        check(_lib.lib().kvc_encode_result(_ptr(result), encoded_cap, C.byref(total), C.byref(max_tile), C.byref(max_stream),
                                           C.byref(tiles), _stream(result)))
    return total.value, max_tile.value, max_stream.value, tiles.value


def k_entropy_encode_cuda_export(input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data,
                                 base_global_offset: int, head_num: int, head_dim: int):
    """src/kernels.cu:919-966.  Returns views (payload, block_infos, thread_infos) of the caller's scratch."""
    return _entropy_encode(True, input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data,
                           base_global_offset, head_num, head_dim)


def v_entropy_encode_cuda_export(input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data,
                                 base_global_offset: int, head_num: int, head_dim: int):
    """src/kernels.cu:968-1011."""
    return _entropy_encode(False, input, encode_code_book, block_infos, thread_infos, idx_offset, encoded_data,
                           base_global_offset, head_num, head_dim)


def _entropy_decode(is_k, in_tensor, block_infos, thread_infos, decode_code_book, out, head_num, head_dim, tree_format):
    for t, n in ((in_tensor, "in_tensor"), (block_infos, "block_infos"), (thread_infos, "thread_infos"),
                 (decode_code_book, "decode_code_book"), (out, "out")):
        _dev_u8(t, n)
    tokens, stride = _geometry(out)
    ms = C.c_float(0.0)
    fn = _lib.lib().kvc_k_entropy_decode if is_k else _lib.lib().kvc_v_entropy_decode
    with torch.cuda.device(out.device):
        check(fn(_ptr(in_tensor), in_tensor.numel(), _ptr(block_infos), block_infos.numel(), _ptr(thread_infos),
                 thread_infos.numel(), _ptr(decode_code_book), decode_code_book.numel(), tree_format, _ptr(out),
                 tokens, stride, head_num, head_dim, C.byref(ms), _stream(out)))
    return float(ms.value)


def k_entropy_decode_cuda_export(in_tensor, block_infos, thread_infos, decode_code_book, out, head_num: int,
                                 head_dim: int, tree_format: int = TREE_I8) -> float:
    """src/kernels.cu:1013-1049.  Writes uint8 symbols into `out` [NB,BS,B,H,D]; returns kernel milliseconds."""
    return _entropy_decode(True, in_tensor, block_infos, thread_infos, decode_code_book, out, head_num, head_dim, tree_format)


def v_entropy_decode_cuda_export(in_tensor, block_infos, thread_infos, decode_code_book, out, head_num: int,
                                 head_dim: int, tree_format: int = TREE_I8) -> float:
    """src/kernels.cu:1051-1087."""
    return _entropy_decode(False, in_tensor, block_infos, thread_infos, decode_code_book, out, head_num, head_dim, tree_format)


def decode_dequant(is_k: bool, in_tensor, block_infos, thread_infos, decode_code_book, quant_min_ints, quant_scales,
                   quant_mask: int, block_size: int, out: torch.Tensor, tree_format: int = TREE_I8) -> float:
    """Huffman decode + (sym + min) * scale in one kernel (models/cache/kvcomp_encode.py:153-166 without the
    uint8 tensor in between).  out: device fp16 [T, B, H, D]; returns elapsed milliseconds."""
    for t, n in ((in_tensor, "in_tensor"), (block_infos, "block_infos"), (thread_infos, "thread_infos"),
                 (decode_code_book, "decode_code_book")):
        _dev_u8(t, n)
    _require(out.is_cuda and out.dtype == torch.float16 and out.dim() == 4 and out.is_contiguous(),
             "out must be a contiguous device float16 tensor [T, B, H, D]")
    _require(quant_min_ints.dtype == torch.int8 and quant_scales.dtype == torch.float16, "min_ints int8, scales fp16")
    T, B, H, D = out.shape
    # the kernel takes the quantization parameters by pointer: they must cover every group of the stream
    groups = _lib.lib().kvc_quant_groups(T // block_size, block_size, B, H, D, quant_mask) if block_size > 0 and T % block_size == 0 else -1
    _require(quant_min_ints.numel() == groups and quant_scales.numel() == groups,
             "%d minima and %d scales for %d quantization groups" % (quant_min_ints.numel(), quant_scales.numel(), groups))
    ms = C.c_float(0.0)
    with torch.cuda.device(out.device):
        check(_lib.lib().kvc_decode_dequant(int(is_k), _ptr(in_tensor), in_tensor.numel(), _ptr(block_infos), block_infos.numel(),
                                            _ptr(thread_infos), thread_infos.numel(), _ptr(decode_code_book),
                                            decode_code_book.numel(), tree_format, _ptr(quant_min_ints.contiguous()),
                                            _ptr(quant_scales.contiguous()), quant_mask, block_size, _ptr(out), T, B, H, D,
                                            C.byref(ms), _stream(out)))
    return ms.value


def _fused(is_k, decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints, quant_scales, B, Cout,
           head_num, head_dim, tree_format):
    for t, n in ((decode_code_book, "decode_code_book"), (block_infos, "block_infos"), (thread_infos, "thread_infos"),
                 (encoded_data, "encoded_data")):
        _dev_u8(t, n)
    _require(quant_min_ints.dtype == torch.int8 and quant_min_ints.is_contiguous(), "quant_min_ints must be contiguous int8")
    _require(quant_scales.dtype == torch.float16 and quant_scales.is_contiguous(), "quant_scales must be contiguous float16")
    _require(B.dtype == torch.float16 and B.is_contiguous() and B.dim() == 3, "B must be a contiguous 3-D float16 tensor")
    _require(Cout.dtype == torch.float16 and Cout.is_contiguous(), "C must be a contiguous float16 tensor")
    batch, q_heads = B.shape[0], B.shape[1]
    if is_k:
        _require(Cout.dim() == 3 and Cout.shape[0] == batch and Cout.shape[1] == q_heads, "C must be [batch, heads, ctx]")
        _require(B.shape[2] == head_dim, "B must be [batch, heads, head_dim]")
        tokens = Cout.shape[2]
        rows = tokens // K_VEC_PER_BLK
        n = quant_scales.numel()
        if n == rows:
            mask = MASK_K_BLOCK
        elif n == rows * batch * head_num * head_dim:
            mask = MASK_CHANNEL
        else:
            raise KvcompError("quant_scales has %d elements: expected one per 64-token block (%d) or one per "
                              "(block, batch, head, channel) (%d)" % (n, rows, rows * batch * head_num * head_dim))
    else:
        tokens = B.shape[2]
        _require(Cout.dim() == 4 and Cout.shape[0] * V_VEC_LEN == tokens and Cout.shape[1] == batch
                 and Cout.shape[2] == q_heads and Cout.shape[3] == head_dim, "C must be [ctx/128, batch, heads, head_dim]")
        n = quant_scales.numel()
        if n == tokens:
            mask = MASK_V_TOKEN
        elif n == tokens * batch:
            mask = MASK_SIM_TOKEN
        elif n == tokens * batch * head_num:
            mask = MASK_VECTOR
        else:
            raise KvcompError("quant_scales has %d elements: expected one per token (%d), per (token, batch) or per "
                              "(token, batch, head)" % (n, tokens))
    _require(quant_min_ints.numel() == n, "quant_min_ints and quant_scales must have the same number of elements")
    ms = C.c_float(0.0)
    fn = _lib.lib().kvc_k_decode_and_mat_vec_mul if is_k else _lib.lib().kvc_v_decode_and_mat_vec_mul
    with torch.cuda.device(B.device):
        check(fn(_ptr(decode_code_book), decode_code_book.numel(), tree_format, _ptr(block_infos), block_infos.numel(),
                 _ptr(thread_infos), thread_infos.numel(), _ptr(encoded_data), encoded_data.numel(),
                 _ptr(quant_min_ints), _ptr(quant_scales), mask, _ptr(B), _ptr(Cout), tokens, batch, head_num, q_heads,
                 head_dim, C.byref(ms), _stream(B)))
    return float(ms.value)


def k_decode_and_mat_vec_mul_cuda_export(decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints,
                                         quant_scales, B, C, head_num: int, head_dim: int,
                                         tree_format: int = TREE_I8) -> float:
    """src/kernels.cu:1093-1136.  C[b,h,t] = sum_i dequant(K)[t,b,h,i] * B[b,h,i]; returns kernel milliseconds."""
    return _fused(True, decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints, quant_scales, B, C,
                  head_num, head_dim, tree_format)


def v_decode_and_mat_vec_mul_cuda_export(decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints,
                                         quant_scales, B, C, head_num: int, head_dim: int,
                                         tree_format: int = TREE_I8) -> float:
    """src/kernels.cu:1138-1180.  C[g,b,h,d] = sum_{t<128} dequant(V)[128g+t,b,h,d] * B[b,h,128g+t]."""
    return _fused(False, decode_code_book, block_infos, thread_infos, encoded_data, quant_min_ints, quant_scales, B, C,
                  head_num, head_dim, tree_format)


def k_mat_vec_mul_cuda_export(k: torch.Tensor, q: torch.Tensor, out: torch.Tensor) -> float:
    """src/kernels.cu:1221-1273: dense fp16 baseline, out[t,b,h] = sum_i k[t,b,h,i] * q[b,h,i]."""
    _require(k.dim() == 4 and q.dim() == 3 and out.dim() == 3, "k [ctx,B,H,D], q [B,H,D], out [ctx,B,H]")
    ctx, batch, heads, dim = k.shape
    _require(q.shape[0] == batch, "Batch size of A and B must be equal")
    _require(q.shape[1] == heads, "Head num of A and B must be equal")
    _require(q.shape[2] == dim, "Head dim of A and B must be equal")
    _require(tuple(out.shape) == (ctx, batch, heads), "out must be [ctx, batch, heads]")
    for t, n in ((k, "A"), (q, "B"), (out, "C")):
        _require(t.dtype == torch.float16, "%s must be of type half" % n)
        _require(t.is_contiguous(), "%s must be contiguous" % n)
    ms = C.c_float(0.0)
    with torch.cuda.device(k.device):
        check(_lib.lib().kvc_k_mat_vec_mul(_ptr(k), _ptr(q), _ptr(out), ctx, batch, heads, dim, C.byref(ms), _stream(k)))
    return float(ms.value)
