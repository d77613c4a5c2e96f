"""The reference's model-facing cache classes, backed by libkvcomp_hip.

    KVCompCachePytorchQuant  <- models/cache/kvcomp_quant.py:14-124   (simulated quantization, what the models run)
    KVCompCache              <- models/cache/kvcomp_cache.py:22-38    (the facade the models construct)
    KVCompCacheCuda          <- models/cache/kvcomp_encode.py:328-368 (entropy-coded storage, one KVCompCtx per layer)

Same constructor `(batch_size, head_num, head_dim, layer_num)`, same `update(key_states, value_states, layer_idx,
cache_kwargs) -> (K, V)` with `[B, H, T, D]` tensors, same `get_seq_length(layer_idx)`, same per-layer lists
(`compressed_{k,v}_cache`, `{k,v}_cache_buffer`, `coss`, `sins`).  The classes do not derive from
`transformers.Cache` (its constructor changed incompatibly after the version the reference pins); they only
implement the two methods a model calls.

Differences in how, not what:
  * the reference re-concatenates the whole history on every step (`safe_cat(..., dim=2)` twice per tensor);
    here each layer owns one dense buffer that grows geometrically, new tokens are appended in place, blocks that
    leave the tail are overwritten in place by their simulated-quantization values, and `update` returns a view.
    The returned tensors therefore alias the cache (strides of the capacity, not of T) and must not be written.
  * the quantize -> dequantize chain of `quant_error` is one kernel (`kvc_quant_error`) instead of ~10 PyTorch
    ops; results are bit-identical.
  * `get_seq_length(None)` returns the length of layer 0 in every mode (the reference's quantized branch computes
    it and drops it, kvcomp_quant.py:119-120), and `KVCompCacheCuda.get_seq_length` returns the stored token
    count (the reference reads `shape[2]` of a `[T, B, H, D]` shape, which is the head count,
    kvcomp_encode.py:362-368).
"""
from typing import Any, Dict, List, Optional, Tuple

import torch

from .compute import apply_rotary_pos_emb_single, blocks_to_compress, quant_dequant_sim, safe_cat
from .ctx import KVCompCacheConfigStatic, KVCompCtx


class JumpOutException(Exception):
    """utils/util.py: raised to leave generation once the caches of the requested round are collected."""


def _config():
    if KVCompCacheConfigStatic.config is None:
        raise ValueError("TComCacheConfigStatic.config is not set. Please set it before using TComCache.")
    return KVCompCacheConfigStatic.config


class _DenseHistory:
    """fp16 [B, H, capacity, D] with the first `length` tokens valid; grows by doubling."""

    def __init__(self):
        self.data: Optional[torch.Tensor] = None
        self.length = 0
        self.quantized = 0        # leading tokens already replaced by their simulated-quantization values

    def append(self, t: torch.Tensor):
        n = t.shape[2]
        if self.data is None or self.length + n > self.data.shape[2]:
            cap = max(2 * (self.length + n), 256)
            grown = torch.empty(t.shape[0], t.shape[1], cap, t.shape[3], dtype=t.dtype, device=t.device)
            if self.data is not None:
                grown[:, :, :self.length].copy_(self.data[:, :, :self.length])
            self.data = grown
        self.data[:, :, self.length:self.length + n].copy_(t)
        self.length += n

    def quantize_blocks(self, block_size, recent_size, eb, mode):
        n = blocks_to_compress(self.length - self.quantized, block_size, recent_size)
        if n > 0:
            region = self.data[:, :, self.quantized:self.quantized + n * block_size]
            region.copy_(quant_dequant_sim(region, block_size, eb, mode))
            self.quantized += n * block_size

    def view(self, lo=0, hi=None, empty_is_none=False):
        hi = self.length if hi is None else hi
        if self.data is None or (empty_is_none and hi <= lo):
            return None
        return self.data[:, :, lo:hi]


class KVCompCachePytorchQuant:
    """models/cache/kvcomp_quant.py:14-124."""
    round_ = 0

    def __init__(self, batch_size, head_num, head_dim, layer_num):
        KVCompCachePytorchQuant.round_ += 1
        self.batch_size = batch_size
        self.head_num = head_num
        self.head_dim = head_dim
        self.compressed_k_cache: List[Optional[torch.Tensor]] = [None] * layer_num
        self.compressed_v_cache: List[Optional[torch.Tensor]] = [None] * layer_num
        self.k_cache_buffer: List[Optional[torch.Tensor]] = [None] * layer_num
        self.v_cache_buffer: List[Optional[torch.Tensor]] = [None] * layer_num
        self.coss: List[Optional[torch.Tensor]] = [None] * layer_num
        self.sins: List[Optional[torch.Tensor]] = [None] * layer_num
        self._k = [_DenseHistory() for _ in range(layer_num)]
        self._v = [_DenseHistory() for _ in range(layer_num)]

    # -- helpers ---------------------------------------------------------------------------------------
    def _rope_in(self, key_states, layer_idx, cache_kwargs):
        cos, sin = cache_kwargs['cos'], cache_kwargs['sin']
        if _config().enable_pre_rope:                  # keys are stored un-rotated, the angles beside them
            self.coss[layer_idx] = safe_cat(self.coss[layer_idx], cos, dim=1)
            self.sins[layer_idx] = safe_cat(self.sins[layer_idx], sin, dim=1)
            return key_states
        return apply_rotary_pos_emb_single(key_states, cos, sin)

    def _publish(self, layer_idx):
        k, v = self._k[layer_idx], self._v[layer_idx]
        # (the reference's compressed caches stay None until a block has been quantized; its tails can be empty)
        self.compressed_k_cache[layer_idx] = k.view(0, k.quantized, empty_is_none=True)
        self.compressed_v_cache[layer_idx] = v.view(0, v.quantized, empty_is_none=True)
        self.k_cache_buffer[layer_idx] = k.view(k.quantized)
        self.v_cache_buffer[layer_idx] = v.view(v.quantized)
        keys = k.view()
        if _config().enable_pre_rope:
            keys = apply_rotary_pos_emb_single(keys, self.coss[layer_idx], self.sins[layer_idx])
        return keys, v.view()

    # -- the Cache contract ------------------------------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        cfg = _config()
        if KVCompCacheConfigStatic.extract_cache is not None:
            assert not cfg.enable_quant, "Disable quant to enable cache collect."
        if cfg.enable_quant is False:
            return self.update_disable(key_states, value_states, layer_idx, cache_kwargs)
        key_states = self._rope_in(key_states, layer_idx, cache_kwargs)
        k, v = self._k[layer_idx], self._v[layer_idx]
        k.append(key_states)
        v.append(value_states)
        k.quantize_blocks(cfg.k_block_size, cfg.k_recent_size, cfg.k_quant_scale_rel, cfg.k_quant_mode)
        v.quantize_blocks(cfg.v_block_size, cfg.v_recent_size, cfg.v_quant_scale_rel, cfg.v_quant_mode)
        return self._publish(layer_idx)

    def update_disable(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
                       cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        key_states = self._rope_in(key_states, layer_idx, cache_kwargs)
        self._k[layer_idx].append(key_states)
        self._v[layer_idx].append(value_states)
        keys, values = self._publish(layer_idx)
        ex = KVCompCacheConfigStatic.extract_cache
        if ex is not None:                              # kvcomp_quant.py:92-100
            rnd = KVCompCachePytorchQuant.round_
            if key_states.shape[2] != 1 and rnd > ex.collect_round:
                raise JumpOutException("\nExtracting cache and new generation round has been detected, "
                                       "jump out to process cache.")
            ex.key_caches.setdefault(rnd - 1, {})
            ex.value_caches.setdefault(rnd - 1, {})
            ex.key_caches[rnd - 1][layer_idx - 1] = self.k_cache_buffer[layer_idx]
            ex.value_caches[rnd - 1][layer_idx - 1] = self.v_cache_buffer[layer_idx]
        return keys, values

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        _config()
        return self._k[0 if layer_idx is None else layer_idx].length


class KVCompCacheCuda:
    """models/cache/kvcomp_encode.py:328-368: every layer keeps an entropy-coded K and V context; `update`
    stores the new tokens and returns the fully decoded history."""
    round_ = 0

    def __init__(self, batch_size, head_num, head_dim, layer_num):
        KVCompCacheCuda.round_ += 1
        cfg = _config()
        self.batch_size = batch_size
        self.head_num = head_num
        self.head_dim = head_dim
        self.k_cache_buffer = [KVCompCtx(True, batch_size, head_num, head_dim, cfg.k_quant_scale_rel) for _ in range(layer_num)]
        self.v_cache_buffer = [KVCompCtx(False, batch_size, head_num, head_dim, cfg.v_quant_scale_rel) for _ in range(layer_num)]
        for ctx in self.k_cache_buffer + self.v_cache_buffer:
            ctx.codebook_smoothing = True        # tokens generated later may quantize to symbols the prompt never produced
            ctx.async_store = True               # appended blocks are encoded without waiting for the device

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        cos, sin = cache_kwargs['cos'], cache_kwargs['sin']
        key_states = apply_rotary_pos_emb_single(key_states, cos, sin)
        self.k_cache_buffer[layer_idx].store(key_states.permute(2, 0, 1, 3), want_symbols=False)
        self.v_cache_buffer[layer_idx].store(value_states.permute(2, 0, 1, 3), want_symbols=False)
        # (get() returns (tensor, milliseconds); the reference permutes the pair itself, kvcomp_encode.py:357-358)
        k_t = self.k_cache_buffer[layer_idx].get()[0].permute(1, 2, 0, 3)
        v_t = self.v_cache_buffer[layer_idx].get()[0].permute(1, 2, 0, 3)
        return k_t, v_t

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.k_cache_buffer[0 if layer_idx is None else layer_idx].ctx_len


class KVCompCache:
    """models/cache/kvcomp_cache.py:22-38: the facade the model code constructs.  `backend` chooses the
    implementation the reference switches by editing a line (kvcomp_cache.py:25-26): "quant" (default, as in
    the reference) or "encode"."""

    def __init__(self, batch_size, head_num, head_dim, layer_num, backend: str = "quant"):
        if backend == "quant":
            self.cache_instance = KVCompCachePytorchQuant(batch_size, head_num, head_dim, layer_num)
        elif backend == "encode":
            self.cache_instance = KVCompCacheCuda(batch_size, head_num, head_dim, layer_num)
        else:
            raise ValueError("backend must be 'quant' or 'encode'")

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        return self.cache_instance.update(key_states, value_states, layer_idx, cache_kwargs)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.cache_instance.get_seq_length(layer_idx)
