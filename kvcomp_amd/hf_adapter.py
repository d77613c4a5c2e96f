"""Compressed KV cache for stock `transformers` models (>= 4.54 / 5.x cache layout: a `Cache` is a list of
per-layer objects).

The reference ships forks of the Llama / Mistral / Phi-3 modelling files pinned to transformers 4.50
(models/llama.py, mistral.py, phi3.py) whose attention layers call `past_key_value.update(k, v, layer_idx,
{"cos", "sin"})` on a `Cache` subclass built with a bare `super().__init__()` (models/cache/kvcomp_encode.py:328-368);
neither the import nor that constructor survives in current releases.  This adapter offers the same behaviour
to unmodified models: every layer keeps one KVCompCtx for K and one for V, `update` appends the new (already
rotated) keys and the values, recompresses the whole blocks that leave the uncompressed tails, and returns the
full dense K and V `[B, H, T, D]` -- decompressed + tail -- exactly what KVCompCacheCuda.update returns
(kvcomp_encode.py:345-360).  `attend` runs decode attention on the compressed form instead, for callers that
bring their own attention loop.

    KVCompCacheConfigStatic.config = KVCompCacheConfig(...)          # as for the reference
    cache = KVCompHFCache(num_layers)
    out = model(input_ids, past_key_values=cache, use_cache=True)
"""
from typing import Optional, Tuple

import torch
from transformers.cache_utils import Cache, CacheLayerMixin

from .attention import CompressedAttention
from .ctx import KVCompCacheConfigStatic, KVCompCtx


class KVCompLayer(CacheLayerMixin):
    """One layer's compressed K and V streams behind the per-layer cache interface."""

    is_sliding = False
    is_compileable = False

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        self.k_ctx: Optional[KVCompCtx] = None
        self.v_ctx: Optional[KVCompCtx] = None
        self._attention: Optional[CompressedAttention] = None

    def lazy_initialization(self, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        cfg = KVCompCacheConfigStatic.config
        assert cfg is not None and cfg.enable_quant, "set KVCompCacheConfigStatic.config (enable_quant=True) first"
        assert key_states.dtype == torch.float16, "the compressed cache stores float16"
        B, H, _, D = key_states.shape
        self.dtype, self.device = key_states.dtype, key_states.device
        self.k_ctx = KVCompCtx(True, B, H, D, cfg.k_quant_scale_rel)
        self.v_ctx = KVCompCtx(False, B, H, D, cfg.v_quant_scale_rel)
        # the codebook comes from the prompt's first blocks; later tokens may quantize to symbols not seen there
        self.k_ctx.codebook_smoothing = self.v_ctx.codebook_smoothing = True
        self.is_initialized = True

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, *args, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        """key_states / value_states [B, H, T_new, D] (keys already rotated) -> dense (K, V) [B, H, T, D]."""
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        self.k_ctx.store(key_states.permute(2, 0, 1, 3).contiguous(), want_symbols=False)
        self.v_ctx.store(value_states.permute(2, 0, 1, 3).contiguous(), want_symbols=False)
        self.keys = self.k_ctx.get()[0].permute(1, 2, 0, 3)
        self.values = self.v_ctx.get()[0].permute(1, 2, 0, 3)
        return self.keys, self.values

    def attend(self, query: torch.Tensor, softmax_scale: Optional[float] = None) -> torch.Tensor:
        """Decode attention of one query per head, `query` [B, H_q, D] fp16 -> fp32 [B, H_q, D], computed on the
        compressed streams (scores, softmax and weighted values fused with the Huffman decode)."""
        assert self.is_initialized and self.get_seq_length() > 0, "the layer holds no tokens"
        if self._attention is None:
            self._attention = CompressedAttention(self.k_ctx, self.v_ctx)
        return self._attention.attend(query, softmax_scale)

    def get_seq_length(self) -> int:
        return 0 if not self.is_initialized else self.k_ctx.ctx_len

    def get_mask_sizes(self, query_length: int) -> Tuple[int, int]:
        return self.get_seq_length() + query_length, 0

    def get_max_length(self) -> int:
        return -1

    def compressed_bytes(self) -> int:
        """Bytes the layer holds: compressed streams plus the fp16 tails."""
        total = 0
        for ctx in (self.k_ctx, self.v_ctx):
            if ctx is None:
                continue
            if ctx.compressed_ctx_len:
                total += ctx.compressed_bytes()
            if ctx.buffer is not None:
                total += ctx.buffer.numel() * 2
        return total

    # the dense tensors handed out by update() are temporaries: nothing to move, clear or reorder in place
    def offload(self):
        pass

    def prefetch(self):
        pass

    def reset(self) -> None:
        self.k_ctx = self.v_ctx = self._attention = None
        self.keys = self.values = None
        self.is_initialized = False

    def reorder_cache(self, beam_idx: torch.LongTensor) -> None:
        raise NotImplementedError("beam search would have to re-encode the streams; use greedy or sampling decoding")

    def crop(self, tokens_to_remove: int) -> None:
        raise NotImplementedError("a compressed stream cannot be cropped in place")


class KVCompHFCache(Cache):
    """`Cache` of KVCompLayer objects; one per decoder layer, or grown on demand when `num_layers` is None."""

    def __init__(self, num_layers: Optional[int] = None):
        if num_layers is None:
            super().__init__(layer_class_to_replicate=KVCompLayer)
        else:
            super().__init__(layers=[KVCompLayer() for _ in range(num_layers)])

    def attend(self, layer_idx: int, query: torch.Tensor, softmax_scale: Optional[float] = None) -> torch.Tensor:
        return self.layers[layer_idx].attend(query, softmax_scale)

    def compressed_bytes(self) -> int:
        return sum(layer.compressed_bytes() for layer in self.layers)

    def compression_ratio(self) -> float:
        """fp16 bytes of everything cached / bytes actually held."""
        dense = 0
        for layer in self.layers:
            if layer.is_initialized:
                c = layer.k_ctx
                dense += 2 * 2 * c.ctx_len * c.batch_size * c.head_num * c.head_dim
        held = self.compressed_bytes()
        return dense / held if held else 1.0
