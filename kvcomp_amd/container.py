"""On-disk / on-wire container of one compressed K or V stream (a KVCompCtx).

The reference keeps compressed caches in process memory only and has no persistent form (its only files are
the two codebook tensors of models/cache/kvcomp_encode.py:46-55).  This container holds everything a decoder
needs, in the reference's own wire format, so a prefilled cache can be stored once and attended to many times:

    bytes 0..7     magic  b"KVCOMP1\\n"
    bytes 8..15    u64 little-endian: length L of the header
    bytes 16..16+L JSON header (utf-8): geometry, quantizer, counters, and for every section its name, dtype,
                   shape, byte offset (from the start of the file, 64-byte aligned) and byte length
    sections       encode_codebook   u8   {u32 code; u32 length} per symbol       (include/huffman.h:13-16)
                   decode_codebook   u8   3-byte (or 5-byte) tree nodes           (include/huffman.h:18-22)
                   block_infos       u8   {u32 offset; u16 byte_num; u16 0} / tile (include/kernels.h:25-28)
                   thread_infos      u8   u16 end_byte * 8 + pad per vector       (include/kernels.h:30-32)
                   quant_min_ints    i8   per quantization group
                   quant_scales      f16  per quantization group
                   encoded_data      u8   tile payloads, MSB-first code bits
                   tail              f16  the uncompressed most recent tokens [t, B, H, D]

Everything is little-endian; nothing in the file is executable or pickled.  `dumps` / `loads` work on bytes,
`save` / `load` on paths.  Loading needs the same process-wide cache configuration (block sizes, recent sizes,
quantization modes) that was in force when the stream was written; the header records it and `load` checks it.
"""
import io
import json
import struct
from typing import Optional

import numpy as np
import torch

from .compute import expected_groups
from .ctx import KVCompCacheConfigStatic, KVCompCtx

MAGIC = b"KVCOMP1\n"
ALIGN = 64
_DTYPES = {"u8": (torch.uint8, np.uint8), "i8": (torch.int8, np.int8), "f16": (torch.float16, np.float16)}


class ContainerError(ValueError):
    pass


def _sections(ctx: KVCompCtx):
    tail = ctx.buffer
    yield "encode_codebook", "u8", ctx.encode_codebook
    yield "decode_codebook", "u8", ctx.decode_codebook
    yield "block_infos", "u8", ctx.block_infos
    yield "thread_infos", "u8", ctx.thread_infos
    yield "quant_min_ints", "i8", ctx.quant_min_ints
    yield "quant_scales", "f16", ctx.quant_scales
    yield "encoded_data", "u8", ctx.encoded_data
    yield "tail", "f16", tail if tail is not None and tail.shape[0] > 0 else None


def dumps(ctx: KVCompCtx) -> bytes:
    """Serialise a context (compressed part, codebooks, quantization metadata, uncompressed tail)."""
    cfg = KVCompCacheConfigStatic.config
    header = {
        "format": 1,
        "is_k": bool(ctx.is_k), "batch_size": ctx.batch_size, "head_num": ctx.head_num, "head_dim": ctx.head_dim,
        "quant_scale_rel": float(ctx.quant_scale_rel), "quant_dims": [int(d) for d in ctx.quant_dims],
        "block_size": ctx.block_size, "recent_size": ctx.recent_size,
        "ctx_len": ctx.ctx_len, "compressed_ctx_len": ctx.compressed_ctx_len,
        "tree_format": ctx.tree_format, "max_code_bits": ctx.max_code_bits, "max_tile_bytes": ctx.max_tile_bytes, "max_stream_bytes": ctx.max_stream_bytes,
        "config": str(cfg) if cfg is not None else None,
        "sections": [],
    }
    blobs = []
    for name, dt, t in _sections(ctx):
        if t is None:
            header["sections"].append({"name": name, "dtype": dt, "shape": None, "offset": 0, "nbytes": 0})
            continue
        a = t.detach().contiguous().cpu().numpy()
        assert a.dtype == _DTYPES[dt][1], (name, a.dtype)
        blobs.append(a.tobytes())
        header["sections"].append({"name": name, "dtype": dt, "shape": list(a.shape), "offset": None, "nbytes": len(blobs[-1])})
    # offsets depend on the header's own length: lay out with a fixed-width placeholder first
    def render(h):
        return json.dumps(h, sort_keys=True).encode("utf-8")
    for sec in header["sections"]:
        if sec["offset"] is None:
            sec["offset"] = 10 ** 15                       # widest value an offset can take here
    hlen = len(render(header)) + 64                        # room for the real (shorter) numbers, padded with spaces
    pos = -(-(16 + hlen) // ALIGN) * ALIGN
    for sec in header["sections"]:
        if sec["nbytes"]:
            sec["offset"] = pos
            pos = -(-(pos + sec["nbytes"]) // ALIGN) * ALIGN
    body = render(header)
    assert len(body) <= hlen
    body = body + b" " * (hlen - len(body))
    out = io.BytesIO()
    out.write(MAGIC)
    out.write(struct.pack("<Q", hlen))
    out.write(body)
    it = iter(blobs)
    for sec in header["sections"]:
        if sec["nbytes"]:
            out.write(b"\0" * (sec["offset"] - out.tell()))
            out.write(next(it))
    return out.getvalue()


def parse_header(data: bytes) -> dict:
    """Header of a container, after validating magic, lengths and section bounds (no tensor is built)."""
    if len(data) < 16 or data[:8] != MAGIC:
        raise ContainerError("not a KVCOMP1 container")
    (hlen,) = struct.unpack("<Q", data[8:16])
    if hlen > len(data) - 16 or hlen > (1 << 24):
        raise ContainerError("header length %d exceeds the data" % hlen)
    try:
        header = json.loads(data[16:16 + hlen].decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise ContainerError("unreadable header: %s" % e)
    if header.get("format") != 1:
        raise ContainerError("unknown container format %r" % header.get("format"))
    for sec in header.get("sections", []):
        if sec["dtype"] not in _DTYPES:
            raise ContainerError("section %s has unknown dtype %r" % (sec["name"], sec["dtype"]))
        if sec["nbytes"]:
            item = np.dtype(_DTYPES[sec["dtype"]][1]).itemsize
            if sec["offset"] % ALIGN or sec["offset"] < 16 + hlen or sec["offset"] + sec["nbytes"] > len(data):
                raise ContainerError("section %s lies outside the data" % sec["name"])
            if int(np.prod(sec["shape"])) * item != sec["nbytes"]:
                raise ContainerError("section %s: shape %s does not match %d bytes" % (sec["name"], sec["shape"], sec["nbytes"]))
    check_consistency(header)
    return header


_SECTION_DTYPES = {"encode_codebook": "u8", "decode_codebook": "u8", "block_infos": "u8", "thread_infos": "u8",
                   "quant_min_ints": "i8", "quant_scales": "f16", "encoded_data": "u8", "tail": "f16"}


def check_consistency(header: dict):
    """The sections must describe one stream of the header's geometry: the kernels take these arrays by pointer, without
    sizes, so a truncated or mismatched array would be read out of bounds on the device."""
    def fail(msg):
        raise ContainerError("inconsistent container: " + msg)
    try:
        is_k = bool(header["is_k"])
        B, H, D = int(header["batch_size"]), int(header["head_num"]), int(header["head_dim"])
        bs, total, comp = int(header["block_size"]), int(header["ctx_len"]), int(header["compressed_ctx_len"])
        dims = [int(d) for d in header["quant_dims"]]
        secs = {sec["name"]: sec for sec in header["sections"]}
    except (KeyError, TypeError, ValueError) as e:
        raise ContainerError("incomplete header: %s" % e)
    if B <= 0 or H <= 0 or D <= 0 or D > 128 or D % 8 or bs <= 0:
        fail("geometry %d x %d x %d, block %d" % (B, H, D, bs))
    tile_tokens = 64 if is_k else 128
    if not 0 <= comp <= total or comp % tile_tokens or comp % bs:
        fail("%d of %d tokens compressed is not a whole number of %d-token tiles and %d-token blocks" % (comp, total, tile_tokens, bs))
    if not is_k and (B * H * D) % 64:
        fail("V rows of %d elements do not split into 64-channel tiles" % (B * H * D))
    for name, dt in _SECTION_DTYPES.items():
        if name not in secs:
            fail("section %s is missing" % name)
        if secs[name]["dtype"] != dt:
            fail("section %s has dtype %s, expected %s" % (name, secs[name]["dtype"], dt))
    def numel(name):
        sec = secs[name]
        return int(np.prod(sec["shape"])) if sec["nbytes"] else 0
    tiles = comp // tile_tokens * (B * H if is_k else B * H * D // 64)
    if numel("block_infos") != tiles * 8:
        fail("block_infos holds %d bytes, %d tiles need %d" % (numel("block_infos"), tiles, tiles * 8))
    if numel("thread_infos") != tiles * 64 * 2:
        fail("thread_infos holds %d bytes, %d tiles need %d" % (numel("thread_infos"), tiles, tiles * 128))
    groups = expected_groups(comp, bs, B, H, D, dims) if comp else 0
    for name in ("quant_min_ints", "quant_scales"):
        if numel(name) != groups:
            fail("%s holds %d values, the stream has %d quantization groups" % (name, numel(name), groups))
    if comp and (not numel("encoded_data") or not numel("decode_codebook") or not numel("encode_codebook")):
        fail("a compressed part without payload or codebook")
    fmt = header.get("tree_format", 3)                     # absent in files written before the field existed: int8 nodes
    if fmt not in (3, 5) or numel("decode_codebook") % fmt:
        fail("decode tree of %d bytes in node format %r" % (numel("decode_codebook"), fmt))
    tail_shape = list(secs["tail"]["shape"]) if secs["tail"]["nbytes"] else [0, B, H, D]
    if tail_shape != [total - comp, B, H, D]:
        fail("the tail has shape %s, expected %s" % (tail_shape, [total - comp, B, H, D]))


def loads(data: bytes, device: Optional[torch.device] = None) -> KVCompCtx:
    """Rebuild a context on `device` (default: the current CUDA device)."""
    header = parse_header(data)
    cfg = KVCompCacheConfigStatic.config
    if cfg is None:
        raise ContainerError("KVCompCacheConfigStatic.config must be set before loading (written with: %s)" % header["config"])
    device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    ctx = KVCompCtx(header["is_k"], header["batch_size"], header["head_num"], header["head_dim"], header["quant_scale_rel"])
    if (ctx.block_size, ctx.recent_size, [int(d) for d in ctx.quant_dims]) != (header["block_size"], header["recent_size"], header["quant_dims"]):
        raise ContainerError("the active cache configuration (block %d, recent %d, dims %s) differs from the one the stream was "
                             "written with (block %d, recent %d, dims %s)" % (ctx.block_size, ctx.recent_size, list(ctx.quant_dims),
                                                                             header["block_size"], header["recent_size"], header["quant_dims"]))
    ctx.device = device
    tensors = {}
    for sec in header["sections"]:
        if not sec["nbytes"]:
            tensors[sec["name"]] = None
            continue
        a = np.frombuffer(data, dtype=_DTYPES[sec["dtype"]][1], count=int(np.prod(sec["shape"])), offset=sec["offset"])
        tensors[sec["name"]] = torch.from_numpy(a.reshape(sec["shape"]).copy()).to(device)
    for name, store in (("encoded_data", ctx._encoded), ("block_infos", ctx._block_infos), ("thread_infos", ctx._thread_infos),
                        ("quant_min_ints", ctx._min_ints), ("quant_scales", ctx._scales)):
        if tensors[name] is not None:
            store.append(tensors[name])
    ctx.encode_codebook = tensors["encode_codebook"]
    ctx.decode_codebook = tensors["decode_codebook"]
    ctx.tree_format = int(header.get("tree_format", 3))
    if tensors["tail"] is not None:
        ctx._tail_append(tensors["tail"])
    ctx.ctx_len = header["ctx_len"]
    ctx.compressed_ctx_len = header["compressed_ctx_len"]
    ctx.max_code_bits = header["max_code_bits"]
    ctx.max_tile_bytes = header["max_tile_bytes"]
    ctx.max_stream_bytes = header["max_stream_bytes"]
    KVCompCtx.buffer_ctx_len.setdefault(device, 0)
    return ctx


def save(ctx: KVCompCtx, path: str):
    with open(path, "wb") as f:
        f.write(dumps(ctx))


def load(path: str, device: Optional[torch.device] = None) -> KVCompCtx:
    with open(path, "rb") as f:
        return loads(f.read(), device)
