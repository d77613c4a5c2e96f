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

A model can also be told to attend on the compressed form by itself: `register_kvcomp_attention()` adds the
attention implementation "kvcomp" to transformers' registry, and a cache built with `attend_compressed=True` then
stops decompressing the history on single-token steps -- `update` stores the token and hands the attention
function a tagged placeholder, the function runs `kvc_attention_decode` over the layer's streams.  Prompts (more
than one query token) still get the dense (K, V) and the stock scaled-dot-product attention.

    register_kvcomp_attention()
    model.set_attn_implementation("kvcomp")
    cache = KVCompHFCache(attend_compressed=True)
    model.generate(input_ids, past_key_values=cache, ...)            # unpadded batches, greedy or sampling
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
        self.attend_compressed = False      # single-token steps: no dense history, the attention function attends here

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
        self.k_ctx.async_store = self.v_ctx.async_store = True      # appended blocks are encoded without waiting for the device
        self.is_initialized = True

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, *args, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        """key_states / value_states [B, H, T_new, D] (keys already rotated) -> dense (K, V) [B, H, T, D]."""
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        self.k_ctx.store(key_states.permute(2, 0, 1, 3).contiguous(), want_symbols=False)
        self.v_ctx.store(value_states.permute(2, 0, 1, 3).contiguous(), want_symbols=False)
        if self.attend_compressed and key_states.shape[2] == 1:
            # kvcomp_attention_forward recognises the tag and attends on the compressed streams of this layer
            key_states._kvcomp_layer = self
            self.keys = self.values = None
            return key_states, value_states
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

    def __init__(self, num_layers: Optional[int] = None, attend_compressed: bool = False):
        self.attend_compressed = attend_compressed
        if num_layers is None:
            super().__init__(layer_class_to_replicate=KVCompLayer)
        else:
            super().__init__(layers=[KVCompLayer() for _ in range(num_layers)])
        for layer in self.layers:
            layer.attend_compressed = attend_compressed

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int, *args, **kwargs):
        while self.attend_compressed and len(self.layers) <= layer_idx:          # layers grown on demand
            self.layers.append(KVCompLayer())
        if self.attend_compressed:
            self.layers[layer_idx].attend_compressed = True
        return super().update(key_states, value_states, layer_idx, *args, **kwargs)

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


def kvcomp_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attention_mask,
                             dropout: float = 0.0, scaling: Optional[float] = None, **kwargs):
    """Attention implementation "kvcomp" for transformers' registry.  A single query token whose key carries the tag
    of a KVCompLayer (see KVCompLayer.update) is answered by decode attention over that layer's compressed streams:
    query [B, H_q, 1, D] -> ([B, 1, H_q, D], None).  Everything else goes to the stock scaled-dot-product attention.
    The compressed path attends over every stored token of every sequence (no padding mask)."""
    layer = getattr(key, "_kvcomp_layer", None)
    if layer is None or query.shape[2] != 1:
        from transformers.integrations.sdpa_attention import sdpa_attention_forward
        return sdpa_attention_forward(module, query, key, value, attention_mask, dropout=dropout, scaling=scaling, **kwargs)
    out = layer.attend(query[:, :, 0, :].contiguous(), scaling)                  # fp32 [B, H_q, D]
    return out.to(query.dtype).unsqueeze(1), None


def register_kvcomp_attention(name: str = "kvcomp") -> str:
    """Make `name` selectable as a model's attention implementation (masks as for "sdpa").  Idempotent."""
    from transformers import AttentionInterface
    from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
    AttentionInterface.register(name, kvcomp_attention_forward)
    AttentionMaskInterface.register(name, sdpa_mask)
    return name
