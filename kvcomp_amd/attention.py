"""Decode attention straight from a compressed KV cache.

The reference stops at two separate kernels (models/cache/kvcomp_encode.py:209-280): raw q.K scores and
per-128-token partial p.V sums that PyTorch adds up; nothing chains them, applies 1/sqrt(d) or softmax, or
handles grouped-query heads (kvcomp_encode.py:328-368 is unreachable code).  This module is that missing
operator: for one layer it owns a K context and a V context (kvcomp_amd.ctx.KVCompCtx) and computes

    out[b, hq] = softmax(q[b, hq] . K[b, hq // rep] / sqrt(d)) . V[b, hq // rep]

over the compressed tokens and the uncompressed tail, with the decoded symbols never written to HBM.
"""
import ctypes as C
import math
from typing import Optional

import torch

from . import _lib, kvcomp_cuda
from ._lib import check
from .compute import dims_to_mask, expected_groups
from .ctx import KVCompCtx


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream(dev):
    return C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def build_lut(decode_codebook: torch.Tensor, tree_format: int = kvcomp_cuda.TREE_I8) -> torch.Tensor:
    """Decode table of one codebook (device uint8 tensor of kvc_lut_bytes() bytes)."""
    L = _lib.lib()
    lut = torch.empty(int(L.kvc_lut_bytes()), dtype=torch.uint8, device=decode_codebook.device)
    with torch.cuda.device(decode_codebook.device):
        check(L.kvc_build_lut(_ptr(decode_codebook), decode_codebook.numel(), tree_format, 1, 0, _ptr(lut),
                              _stream(decode_codebook.device)))
    return lut


def k_scores(ctx: KVCompCtx, lut: torch.Tensor, q: torch.Tensor, out: Optional[torch.Tensor] = None,
             timed: bool = False):
    """fp32 scores [B, Hq, ctx_c] = q . dequant(K) for the compressed part of a K context."""
    B, Hq, D = q.shape
    if out is None:
        out = torch.empty(B, Hq, ctx.compressed_ctx_len, dtype=torch.float32, device=q.device)
    ms = C.c_float(0.0)
    with torch.cuda.device(q.device):
        check(_lib.lib().kvc_k_scores_lut(
            _ptr(lut), 0, _ptr(ctx.block_infos), ctx.block_infos.numel(), _ptr(ctx.thread_infos), ctx.thread_infos.numel(),
            _ptr(ctx.encoded_data), ctx.encoded_data.numel(), _ptr(ctx.quant_min_ints), _ptr(ctx.quant_scales),
            dims_to_mask(ctx.quant_dims), _ptr(q), _ptr(out), 1 if out.dtype == torch.float32 else 0, ctx.max_tile_bytes,
            ctx.max_stream_bytes, ctx.max_code_bits,
            ctx.compressed_ctx_len, B, ctx.head_num, Hq, D, C.byref(ms) if timed else None, _stream(q.device)))
    return out, float(ms.value)


def v_partials(ctx: KVCompCtx, lut: torch.Tensor, p: torch.Tensor, out: Optional[torch.Tensor] = None,
               timed: bool = False):
    """fp32 partial sums [ctx_c / 128, B, Hq, D] of p . dequant(V) for the compressed part of a V context."""
    B, Hq, T = p.shape
    if out is None:
        out = torch.empty(T // kvcomp_cuda.V_VEC_LEN, B, Hq, ctx.head_dim, dtype=torch.float32, device=p.device)
    ms = C.c_float(0.0)
    with torch.cuda.device(p.device):
        check(_lib.lib().kvc_v_partials_lut(
            _ptr(lut), 0, _ptr(ctx.block_infos), ctx.block_infos.numel(), _ptr(ctx.thread_infos), ctx.thread_infos.numel(),
            _ptr(ctx.encoded_data), ctx.encoded_data.numel(), _ptr(ctx.quant_min_ints), _ptr(ctx.quant_scales),
            dims_to_mask(ctx.quant_dims), _ptr(p), _ptr(out), 1 if out.dtype == torch.float32 else 0, ctx.max_tile_bytes,
            ctx.max_stream_bytes, ctx.max_code_bits,
            T, B, ctx.head_num, Hq, ctx.head_dim, C.byref(ms) if timed else None, _stream(p.device)))
    return out, float(ms.value)


class CompressedAttention:
    """Decode attention of one layer over (compressed K, compressed V, uncompressed tails)."""

    def __init__(self, k_ctx: KVCompCtx, v_ctx: KVCompCtx):
        assert k_ctx.is_k and not v_ctx.is_k
        self.k, self.v = k_ctx, v_ctx
        self._k_lut = self._v_lut = None
        self._k_lut_src = self._v_lut_src = None
        self._workspace = None
        self._keep = []

    def _luts(self):
        # decode tables follow the contexts' codebooks (built once, rebuilt if a codebook is replaced)
        # (a context has no codebook until its first block is compressed)
        if self.k.decode_codebook is not None and self._k_lut_src is not self.k.decode_codebook:
            self._k_lut, self._k_lut_src = build_lut(self.k.decode_codebook, self.k.tree_format), self.k.decode_codebook
        if self.v.decode_codebook is not None and self._v_lut_src is not self.v.decode_codebook:
            self._v_lut, self._v_lut_src = build_lut(self.v.decode_codebook, self.v.tree_format), self.v.decode_codebook
        return self._k_lut, self._v_lut

    @staticmethod
    def _bracket(prof, key):
        if prof is None:
            return None
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        prof[key].append((a, b))
        a.record()
        return b

    @staticmethod
    def _bracket_end(ev):
        if ev is not None:
            ev.record()

    def _desc(self, ctx: KVCompCtx, lut) -> "_lib.CompressedDesc":
        d = _lib.CompressedDesc()
        if ctx._probe is not None:
            ctx.poll_stores()                              # what queued stores have left, if it has arrived: no wait
        if ctx.compressed_ctx_len:
            d.d_luts = lut.data_ptr()
            # (addresses and sizes straight from the contexts' growing arrays: a tensor view per field and call costs more
            # host time than a short-context step takes on the device)
            d.d_block_infos, d.block_infos_bytes = ctx._block_infos.address_and_numel()
            d.d_thread_infos, d.thread_infos_bytes = ctx._thread_infos.address_and_numel()
            enc, enc_bytes = ctx.encoded_nosync()          # an address and a bound: no wait for queued encodes
            d.d_encoded, d.encoded_bytes = enc.data_ptr(), enc_bytes
            # the kernels take the quantization parameters by pointer: they must cover every group of the stream
            groups = expected_groups(ctx.compressed_ctx_len, ctx.block_size, ctx.batch_size, ctx.head_num, ctx.head_dim, ctx.quant_dims)
            (d.d_quant_min_ints, n_min), (d.d_quant_scales_f16, n_scale) = ctx._min_ints.address_and_numel(), ctx._scales.address_and_numel()
            assert n_min == groups and n_scale == groups, \
                "the context holds %d minima and %d scales for %d quantization groups" % (n_min, n_scale, groups)
        d.rows_per_codebook = 0
        d.quant_mask = dims_to_mask(ctx.quant_dims)
        d.max_tile_bytes, d.max_stream_bytes, d.max_code_bits = ctx.max_tile_bytes, ctx.max_stream_bytes, ctx.max_code_bits
        d.tokens = ctx.compressed_ctx_len
        tail = ctx.buffer
        d.tail_tokens = 0 if tail is None else tail.shape[0]
        if d.tail_tokens:
            self._keep.append(tail.contiguous())
            d.d_tail_f16 = self._keep[-1].data_ptr()
        return d

    def attend(self, q: torch.Tensor, scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
               kernel_ms: Optional[list] = None) -> torch.Tensor:
        """q fp16 [B, Hq, D] -> fp32 [B, Hq, D] over every stored token, as one library call
        (kvc_attention_decode): scores, softmax and the weighted sum of values never pass through PyTorch.
        `kernel_ms`, if a list, receives (fused K kernel ms, fused V kernel ms) -- which makes the call wait."""
        B, Hq, D = q.shape
        assert q.dtype == torch.float16 and self.v.ctx_len == self.k.ctx_len
        scale = scale if scale is not None else 1.0 / math.sqrt(D)
        k_lut, v_lut = self._luts()
        L = _lib.lib()
        need = int(L.kvc_attention_workspace_bytes(self.k.ctx_len, self.v.compressed_ctx_len, B, Hq, D))
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != q.device:
            self._workspace = torch.empty(need + need // 4, dtype=torch.uint8, device=q.device)
        if out is None:
            out = torch.empty(B, Hq, D, dtype=torch.float32, device=q.device)
        self._keep = []
        kd, vd = self._desc(self.k, k_lut), self._desc(self.v, v_lut)
        q = q.contiguous()
        ms = (C.c_float * 2)()
        with torch.cuda.device(q.device):
            check(L.kvc_attention_decode(C.byref(kd), C.byref(vd), _ptr(q), float(scale), _ptr(self._workspace),
                                         self._workspace.numel(), _ptr(out), B, self.k.head_num, Hq, D, None,
                                         ms if kernel_ms is not None else None, _stream(q.device)))
        if kernel_ms is not None:
            kernel_ms[:] = [float(ms[0]), float(ms[1])]
        return out

    def attend_stepwise(self, q: torch.Tensor, scale: Optional[float] = None, prof: Optional[dict] = None) -> torch.Tensor:
        """The same result assembled from the reference-shaped pieces (fused K scores, PyTorch softmax, fused
        p.V partials, PyTorch reduction).  q fp16 [B, Hq, D] -> fp32 [B, Hq, D].  Covers every stored token: the compressed part through the
        fused kernels, the fp16 tails (K and V compress on different block sizes, so their tails differ)
        through dense matvecs.  `prof`, if given, collects (start, end) event pairs recorded on the launch
        stream around the two fused kernels under the keys "k" and "v"."""
        B, Hq, D = q.shape
        rep = Hq // self.k.head_num
        scale = scale if scale is not None else 1.0 / math.sqrt(D)
        k_lut, v_lut = self._luts()
        T = self.k.ctx_len
        assert self.v.ctx_len == T
        kc, vc = self.k.compressed_ctx_len, self.v.compressed_ctx_len
        parts = []
        if kc:
            ev = self._bracket(prof, "k")
            parts.append(k_scores(self.k, k_lut, q)[0])
            self._bracket_end(ev)
        if kc != T:
            tail = self.k.buffer.float().repeat_interleave(rep, dim=2)                  # [t, B, Hq, D]
            parts.append(torch.einsum("tbhd,bhd->bht", tail, q.float()))
        scores = parts[0] if len(parts) == 1 else torch.cat(parts, dim=-1)
        p = torch.softmax(scores * scale, dim=-1)
        out = torch.zeros(B, Hq, D, dtype=torch.float32, device=q.device)
        if vc:
            p16 = p[:, :, :vc].to(torch.float16).contiguous()
            ev = self._bracket(prof, "v")
            part, _ = v_partials(self.v, v_lut, p16)
            self._bracket_end(ev)
            out += part.sum(dim=0)
        if vc != T:
            tail = self.v.buffer.float().repeat_interleave(rep, dim=2)
            out += torch.einsum("tbhd,bht->bhd", tail, p[:, :, vc:])
        return out
