"""Compressed KV-cache context: the object layout and methods of the reference's KVCompCtx
(models/cache/kvcomp_encode.py:15-326), with every device step running through libkvcomp_hip.

Same attribute names (encoded_data, block_infos, thread_infos, quant_min_ints, quant_scales, encode_codebook,
decode_codebook, buffer, ctx_len, compressed_ctx_len, shape) and the same method contracts (store, get,
get_only_compressed, get_decode_quant_ints, mat_vec_mul, build_codebook, get_cr).  Differences:

  * the quantizer is one HIP launch instead of ~8 fp16 PyTorch kernels (bit-identical symbols);
  * encoder scratch is kept per device and only grows (the reference re-allocates and zero-fills four
    buffers on every store, kvcomp_encode.py:88-95), and the accumulated stream lives in amortised
    growable buffers instead of being re-concatenated on every store (kvcomp_encode.py:129-133);
  * batch > 1 and per-channel K (QuantMode.ChannelQuant) are accepted.
"""
import ast
import math
from typing import Dict, List, Optional, Tuple

import torch

from . import kvcomp_cuda
from ._lib import KvcompError
from .compute import (QUANT_MODE_MAP, QuantMode, blocks_to_compress, cut_tensor_ctx_len_0, dequant, dims_to_mask,  # noqa: F401
                      mask_keepdim_shape, quant, safe_cat)


class ExtractCacheConfig:
    """utils/config.py:3-19"""

    def __init__(self, collect_round: int):
        self.collect_round = collect_round
        self.key_caches = {}
        self.value_caches = {}

    def size(self):
        total = 0
        for caches in (self.key_caches, self.value_caches):
            for per_round in caches.values():
                for t in per_round.values():
                    total += t.numel() * 16
        return total


class KVCompCacheConfig:
    """utils/config.py:21-140: the eleven configuration fields, printable and parseable."""

    _FIELDS = ("enable_quant", "model_name", "enable_pre_rope", "k_quant_mode", "v_quant_mode", "k_block_size",
               "v_block_size", "k_recent_size", "v_recent_size", "k_quant_scale_rel", "v_quant_scale_rel")

    def __init__(self, model_name, k_quant_mode, v_quant_mode, k_block_size, v_block_size, k_recent_size,
                 v_recent_size, k_quant_scale_rel, v_quant_scale_rel, enable_quant=True, enable_pre_rope=False):
        self.enable_quant = enable_quant
        self.model_name = model_name
        self.enable_pre_rope = enable_pre_rope
        self.k_quant_mode = k_quant_mode
        self.v_quant_mode = v_quant_mode
        self.k_block_size = k_block_size
        self.v_block_size = v_block_size
        self.k_recent_size = k_recent_size
        self.v_recent_size = v_recent_size
        self.k_quant_scale_rel = k_quant_scale_rel
        self.v_quant_scale_rel = v_quant_scale_rel

    def __str__(self):
        d = {"enable_quant": self.enable_quant, "enable_pre_rope": self.enable_pre_rope, "model_name": self.model_name}
        if self.enable_quant:
            d.update(k_quant_mode=self.k_quant_mode.value, v_quant_mode=self.v_quant_mode.value,
                     k_block_size=self.k_block_size, v_block_size=self.v_block_size,
                     k_recent_size=self.k_recent_size, v_recent_size=self.v_recent_size,
                     k_quant_scale_rel=self.k_quant_scale_rel, v_quant_scale_rel=self.v_quant_scale_rel)
        return str(d)

    __repr__ = __str__

    @staticmethod
    def from_str(text: str):
        d = ast.literal_eval(text)       # the reference uses eval (utils/config.py:71); literals are all it needs
        if d["enable_quant"]:
            kw = dict(k_quant_mode=QuantMode(d["k_quant_mode"]), v_quant_mode=QuantMode(d["v_quant_mode"]),
                      k_block_size=d["k_block_size"], v_block_size=d["v_block_size"],
                      k_recent_size=d["k_recent_size"], v_recent_size=d["v_recent_size"],
                      k_quant_scale_rel=d["k_quant_scale_rel"], v_quant_scale_rel=d["v_quant_scale_rel"])
        else:
            kw = dict(k_quant_mode=None, v_quant_mode=None, k_block_size=None, v_block_size=None, k_recent_size=None,
                      v_recent_size=None, k_quant_scale_rel=None, v_quant_scale_rel=None)
        return KVCompCacheConfig(model_name=d["model_name"], enable_quant=d["enable_quant"],
                                 enable_pre_rope=d["enable_pre_rope"], **kw)

    def _key(self):
        return tuple(getattr(self, f) for f in self._FIELDS)

    def __eq__(self, other):
        return isinstance(other, KVCompCacheConfig) and self._key() == other._key()

    def __hash__(self):
        return hash(self._key())


class KVCompCacheConfigStatic:
    """Process-wide configuration slot (models/cache/kvcomp_quant.py:10-12)."""
    config: Optional[KVCompCacheConfig] = None
    extract_cache: Optional[ExtractCacheConfig] = None


class _Growable:
    """Device buffer that grows geometrically (by a quarter) along dim 0; `.view` is the filled prefix."""

    def __init__(self):
        self.data: Optional[torch.Tensor] = None
        self.used = 0

    def append(self, t: torch.Tensor):
        n = t.shape[0]
        # room for a quarter more than is needed: re-allocation stays rare while decoding appends small pieces, and a
        # context never holds much more than its stream
        if self.data is None:
            cap = n + max(n // 4, 16)
            self.data = torch.empty((cap,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
        elif self.used + n > self.data.shape[0]:
            cap = self.used + n + max((self.used + n) // 4, 16)
            grown = torch.empty((cap,) + tuple(self.data.shape[1:]), dtype=self.data.dtype, device=self.data.device)
            grown[:self.used] = self.data[:self.used]
            self.data = grown
        self.data[self.used:self.used + n] = t
        self.used += n

    def reserve(self, n: int, tail_shape, dtype, device):
        """Make room for n more rows behind the filled part (which is kept); returns the view of those rows."""
        if self.data is None:
            self.data = torch.empty((n + max(n // 4, 16),) + tuple(tail_shape), dtype=dtype, device=device)
        elif self.used + n > self.data.shape[0]:
            cap = self.used + n + max((self.used + n) // 4, 16)
            grown = torch.empty((cap,) + tuple(self.data.shape[1:]), dtype=self.data.dtype, device=self.data.device)
            grown[:self.used] = self.data[:self.used]
            self.data = grown
        return self.data[self.used:self.used + n]

    def trim(self):
        """Give back what was reserved beyond a quarter of the filled part (after a worst-case reservation)."""
        cap = self.used + max(self.used // 4, 16)
        if self.data is not None and self.data.shape[0] > cap:
            kept = torch.empty((cap,) + tuple(self.data.shape[1:]), dtype=self.data.dtype, device=self.data.device)
            kept[:self.used] = self.data[:self.used]
            self.data = kept

    @property
    def view(self) -> Optional[torch.Tensor]:
        return None if self.data is None else self.data[:self.used]

    def address_and_numel(self):
        """(device address, elements) of the filled part without making a tensor for it (0, 0 while empty)."""
        if self.data is None:
            return 0, 0
        row = 1
        for n in self.data.shape[1:]:
            row *= n
        return self.data.data_ptr(), self.used * row


class KVCompCtx:
    """One compressed K or V stream of one layer (models/cache/kvcomp_encode.py:15-326)."""

    # encoder scratch shared by every context on a device (kvcomp_encode.py:17-21); grown, never shrunk
    buffer_ctx_len: Dict[torch.device, int] = dict()
    block_infos_buffer: Dict[torch.device, torch.Tensor] = dict()
    thread_infos_buffer: Dict[torch.device, torch.Tensor] = dict()
    idx_offset_buffer: Dict[torch.device, torch.Tensor] = dict()
    pre_alloc_compressed_data_buffer: Dict[torch.device, torch.Tensor] = dict()

    def __init__(self, is_k: bool, batch_size: int, head_num: int, head_dim: int, quant_scale_rel: float,
                 encode_codebook_path: str = None, decode_codebook_path: str = None):
        cfg = KVCompCacheConfigStatic.config
        assert cfg is not None, "KVCompCacheConfigStatic.config is None"
        assert cfg.k_quant_mode in (QuantMode.BlockQuant, QuantMode.ChannelQuant), \
            "k_quant_mode must be BlockQuant or ChannelQuant for the kernel implementation"
        assert cfg.v_quant_mode in (QuantMode.TokenQuant, QuantMode.VectorQuant), \
            "v_quant_mode must be TokenQuant or VectorQuant for the kernel implementation"
        assert head_dim <= kvcomp_cuda.K_VEC_LEN and head_dim % 8 == 0, "head_dim must be a multiple of 8, at most K_VEC_LEN"
        self.is_k = is_k
        self.batch_size = batch_size
        self.head_num = head_num
        self.head_dim = head_dim
        self.quant_scale_rel = quant_scale_rel
        self.ctx_len = 0
        self.compressed_ctx_len = 0
        self.device: Optional[torch.device] = None
        self.quant_dims = QUANT_MODE_MAP[cfg.k_quant_mode] if is_k else QUANT_MODE_MAP[cfg.v_quant_mode]
        self.block_size = cfg.k_block_size if is_k else cfg.v_block_size
        self.recent_size = cfg.k_recent_size if is_k else cfg.v_recent_size
        if is_k:
            assert (batch_size * head_num * head_dim) % head_dim == 0
            assert self.block_size == kvcomp_cuda.K_VEC_PER_BLK, "for K, block size must equal VEC_PER_BLK"
        else:
            assert (batch_size * head_num * head_dim) % kvcomp_cuda.V_VEC_PER_BLK == 0, "hidden size must be divisible by VEC_PER_BLK"
            assert self.block_size % kvcomp_cuda.V_VEC_LEN == 0, "block size must be divisible by VEC_LEN"
        self._encoded = _Growable()
        self._block_infos = _Growable()
        self._thread_infos = _Growable()
        self._min_ints = _Growable()
        self._scales = _Growable()
        self._tail: Optional[torch.Tensor] = None      # [capacity, B, H, D]; the first _tail_len tokens are the tail
        self._tail_len = 0
        self.max_code_bits = 0           # longest code of the codebook (0 = unknown)
        self.max_tile_bytes = 0            # largest tile payload seen so far (sizes the fused decoders' LDS staging)
        self.max_stream_bytes = 0          # longest lane stream seen so far (sizes the fused decoders' LDS rows)
        self.encode_codebook: Optional[torch.Tensor] = None
        self.decode_codebook: Optional[torch.Tensor] = None
        # node layout of decode_codebook: the reference's 3-byte nodes (include/huffman.h:18-22) while the code fits them
        # (at most 128 nodes, symbols up to 127), else 5-byte nodes; every decoder of this context is told which
        self.tree_format = kvcomp_cuda.TREE_I8
        # what encodes that nobody waited for have left on the device: words 0 - 7 are kvc_encode_async's result words,
        # word 8 counts the payload bytes in _encoded; _enc_pending bounds the bytes the host has not learnt of yet
        self._state: Optional[torch.Tensor] = None
        self._enc_pending = 0
        # Stores that were queued and not yet seen to succeed, oldest first: (tokens, their fp16 rows or None, the
        # bookkeeping as it stood right after the store, the store's share of _enc_pending, whether the tokens are gone
        # if the store has to be taken back: counted in ctx_len, rows not kept); _verified is the
        # bookkeeping behind the last store that is known to be good.  _probe = (event, stores covered) while a copy of
        # the device words to _host_words (pinned) is on its way: reading it later costs no wait.
        self._unverified: list = []
        self._verified = None
        self._probe = None
        self._host_words: Optional[torch.Tensor] = None
        self._trim_after_sync = False
        self.waits = 0                     # how often this context has waited for the device to learn sizes

    def _device_state(self) -> torch.Tensor:
        if self._state is None:
            self._state = torch.zeros(16, dtype=torch.int32, device=self.device)
            self._state[8] = self._encoded.used
        return self._state

    def _bookkeeping(self):
        return (self._block_infos.used, self._thread_infos.used, self._min_ints.used, self._scales.used, self.compressed_ctx_len)

    def _sync_sizes(self):
        """Learn from the device how many payload bytes the encodes queued so far have produced (waits for them).  If
        one of them failed, every store queued since the last one known to be good is taken back (their tokens return
        to the front of the tail) and the error is raised."""
        if self._enc_pending == 0:
            return
        self.waits += 1
        try:
            _, max_tile, max_stream, _ = kvcomp_cuda.encode_result(self._state[:8], self._encoded.data.numel())
        except KvcompError:
            self._roll_back()
            raise
        self._probe = None
        self._accept(len(self._unverified), int(self._state[8].item()), max_tile, max_stream)

    def _accept(self, n_stores: int, used: int, max_tile: int, max_stream: int):
        """The first n_stores queued stores are done and good; `used` payload bytes lie in _encoded behind them."""
        done, self._unverified = self._unverified[:n_stores], self._unverified[n_stores:]
        self._encoded.used = used
        self._enc_pending = sum(u[3] for u in self._unverified)
        self.max_tile_bytes = max(self.max_tile_bytes, max_tile)
        self.max_stream_bytes = max(self.max_stream_bytes, max_stream)
        if done:
            self._verified = done[-1][2] + (used,)
        if self._trim_after_sync and not self._unverified:
            self._trim_after_sync = False
            self._encoded.trim()                               # a byte per symbol was reserved; the stream is a fraction of it

    def _roll_back(self):
        """Back to the last store that is known to be good: the stores queued since then are dropped from the
        bookkeeping, the device's words say so too, and the tokens of those stores return to the front of the tail
        (rows that were not kept -- stores recorded into a graph -- are lost and leave ctx_len)."""
        if self._verified is None:
            return
        (self._block_infos.used, self._thread_infos.used, self._min_ints.used, self._scales.used, self.compressed_ctx_len,
         self._encoded.used) = self._verified
        st = self._state
        st[1:5] = 0                                            # no error; the size hints start again from the host's
        st[4] = self._block_infos.used // 8
        st[8] = self._encoded.used
        self._enc_pending = 0
        rows = [u[1] for u in self._unverified if u[1] is not None]
        self.ctx_len -= sum(u[0] for u in self._unverified if u[4])
        if rows:
            if self._tail_len:
                rows.append(self._tail[:self._tail_len])
            self._tail = torch.cat(rows, dim=0)
            self._tail_len = self._tail.shape[0]
        self._unverified = []
        self._probe = None

    def _issue_probe(self):
        """Ask for a copy of the device words without waiting for it (nothing is asked for while the stream is being
        recorded into a graph, or while an earlier copy is on its way)."""
        if self._probe is not None or not self._unverified or torch.cuda.is_current_stream_capturing():
            return
        if self._host_words is None:
            self._host_words = torch.empty(16, dtype=torch.int32, pin_memory=True)
        self._host_words.copy_(self._state, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._probe = (ev, len(self._unverified))

    def poll_stores(self):
        """Look, without waiting, at what the stores queued by async_store have left: sizes and size hints are brought
        up to date, and a store that failed on the device is reported here (KvcompError) with the context rolled back to
        the last good store.  Called by store() and by the attention operator; cheap when nothing is outstanding."""
        p = self._probe
        if p is None or not p[0].query():
            return
        w = self._host_words
        if int(w[1]) != 0:
            self._sync_sizes()                                 # takes the stores back and raises, with the library's message
            return
        self._probe = None
        self._accept(p[1], int(w[8]), int(w[2]), int(w[3]))
        self._issue_probe()

    def encoded_nosync(self):
        """(payload buffer, upper bound of the bytes in use) without waiting for queued encodes: for callers that
        only need an address and a bound, like the fused kernels."""
        if self._encoded.data is None:
            return None, 0
        return self._encoded.data, min(self._encoded.used + self._enc_pending, self._encoded.data.numel())

    def _append_encoded(self, encoded_: torch.Tensor):
        self._sync_sizes()
        self._encoded.append(encoded_)
        if self._state is not None:
            self._state[8] = self._encoded.used

    @property
    def encoded_data(self) -> Optional[torch.Tensor]:
        """The reference's attribute (kvcomp_encode.py:56): the payload so far (waits for queued encodes)."""
        self._sync_sizes()
        return self._encoded.view

    @property
    def buffer(self) -> Optional[torch.Tensor]:
        """The uncompressed most recent tokens [t, B, H, D] (kvcomp_encode.py:61); a view of a preallocated area."""
        return None if self._tail is None else self._tail[:self._tail_len]

    def _tail_append(self, cache: torch.Tensor):
        n = cache.shape[0]
        if self._tail is None or self._tail_len + n > self._tail.shape[0]:
            # what a context keeps between stores is less than block_size + recent_size tokens; room for that plus
            # the tokens being appended (single tokens while decoding), with some slack against re-allocation
            cap = self._tail_len + n + self.block_size + 64
            grown = torch.empty((cap,) + tuple(cache.shape[1:]), dtype=cache.dtype, device=cache.device)
            if self._tail_len:
                grown[:self._tail_len] = self._tail[:self._tail_len]
            self._tail = grown
        self._tail[self._tail_len:self._tail_len + n] = cache
        self._tail_len += n

    def _tail_drop_front(self, n: int):
        rest = self._tail_len - n
        if rest > 0:
            src = self._tail[n:self._tail_len]
            self._tail[:rest] = src.clone() if rest > n else src       # overlapping ranges go through a copy
        self._tail_len = rest

    # the reference's public tensor attributes (kvcomp_encode.py:56-61)
    block_infos = property(lambda self: self._block_infos.view)
    thread_infos = property(lambda self: self._thread_infos.view)
    quant_min_ints = property(lambda self: self._min_ints.view)
    quant_scales = property(lambda self: self._scales.view)

    def _check(self, cache: torch.Tensor):
        assert cache.dtype == torch.float16, "cache must be float16"
        assert cache.shape[1] == self.batch_size, "batch size mismatch"
        assert cache.shape[2] == self.head_num, "head num mismatch"
        assert cache.shape[3] == self.head_dim, "head dim mismatch"

    def _scratch(self, sizes):
        dev = self.device
        for store, n in ((KVCompCtx.block_infos_buffer, sizes[0]), (KVCompCtx.thread_infos_buffer, sizes[1]),
                         (KVCompCtx.idx_offset_buffer, sizes[2]), (KVCompCtx.pre_alloc_compressed_data_buffer, sizes[3])):
            if dev not in store or store[dev].numel() < n:
                store[dev] = torch.empty(n, dtype=torch.uint8, device=dev)
        return (KVCompCtx.block_infos_buffer[dev], KVCompCtx.thread_infos_buffer[dev],
                KVCompCtx.idx_offset_buffer[dev], KVCompCtx.pre_alloc_compressed_data_buffer[dev])

    # With a codebook in place, whole blocks can go from fp16 to payload in one library call that never
    # materialises the symbols; callers that do not look at store()'s return value ask for it.
    fused_store = True

    def store(self, cache: torch.Tensor, want_symbols: bool = True):
        """kvcomp_encode.py:69-136: append [T_new, B, H, D]; compress the whole blocks that leave the tail.
        Returns the uint8 symbols that were compressed (None if nothing left the tail, or if want_symbols is
        False and the fused quantize + encode path ran)."""
        self._check(cache)
        if self.device is None:
            self.device = cache.device
        assert self.device == cache.device, "device mismatch"
        if self._probe is not None:
            self.poll_stores()
        # cut_tensor_ctx_len_0 (utils/compute.py:59-72): the leading whole blocks of (tail + new tokens) that leave the
        # recent window are compressed, the rest is the new tail.  The blocks are taken from where they lie (the tail,
        # the incoming tensor, or -- when they span both -- a copy of just those tokens), so a long prompt never passes
        # through the tail and the tail stays a few blocks long.  Nothing of the context changes before the encoder
        # has succeeded: a failed store (a symbol without a code, a tile beyond 8191 bytes) leaves it as it was.
        n_new = cache.shape[0]
        n_blocks = blocks_to_compress(self._tail_len + n_new, self.block_size, self.recent_size)
        if n_blocks <= 0:
            self._tail_append(cache)
            self.ctx_len += n_new
            return None
        n_c = n_blocks * self.block_size
        from_tail = min(n_c, self._tail_len)
        if from_tail == 0:
            to_compress = cache[:n_c].contiguous()
        elif from_tail == n_c:
            to_compress = self._tail[:n_c]
        else:
            to_compress = torch.cat([self._tail[:from_tail], cache[:n_c - from_tail]], dim=0)
        sym = self._compress(to_compress, want_symbols)
        if n_c >= self._tail_len:
            rest = cache[n_c - self._tail_len:]
            self._tail_len = 0
            self._tail_append(rest)
        else:
            self._tail_drop_front(n_c)
            self._tail_append(cache)
        self.ctx_len += n_new
        return sym

    def _compress(self, to_compress: torch.Tensor, want_symbols: bool):
        """Quantize + encode whole blocks [n * block_size, B, H, D] and append the stream; returns the symbols on the
        two-step path.  State is only touched after the library calls have succeeded."""
        mask = dims_to_mask(self.quant_dims)
        if (not want_symbols and KVCompCtx.fused_store and self.async_store and self.encode_codebook is not None
                and kvcomp_cuda.store_fused_supported(self.is_k, mask, self.batch_size, self.head_num, self.head_dim)):
            T = to_compress.shape[0]
            capturing = torch.cuda.is_current_stream_capturing()
            large = T > self.ASYNC_KEEP_BLOCKS * self.block_size
            # the rows of a small store are kept until the store is seen to have succeeded (a copy: the caller's tensor
            # and the tail are both overwritten soon); a large one is waited for here, with its rows still in place
            keep = None if (large or capturing) else to_compress.clone()
            self._encode_direct(T, cache=to_compress, mask=mask, tables=self.encode_codebook,
                                table_bytes=self.encode_codebook.numel(), keep=keep, lost_if_dropped=capturing)
            if large and not capturing:
                self._trim_after_sync = True
                self._sync_sizes()
            else:
                self._issue_probe()
            return None
        if (not want_symbols and KVCompCtx.fused_store and self.encode_codebook is not None
                and kvcomp_cuda.store_fused_supported(self.is_k, mask, self.batch_size, self.head_num, self.head_dim)):
            self._store_fused(to_compress, mask)
            return None
        blocked = to_compress.reshape(-1, self.block_size, self.batch_size, self.head_num, self.head_dim)
        quant_ints, min_ints, quant_scale = quant(blocked, self.quant_dims, self.quant_scale_rel)
        if self.encode_codebook is None and self.device_codebook:
            self._first_chunk_on_device(quant_ints, min_ints, quant_scale)
            return quant_ints
        sizes = kvcomp_cuda.calculate_buffer_size(quant_ints, self.is_k, self.head_num, self.head_dim)
        KVCompCtx.buffer_ctx_len[self.device] = to_compress.shape[0]
        bi_buf, ti_buf, idx_buf, payload_buf = self._scratch(sizes)
        codebook = None
        if self.encode_codebook is None:     # first stored chunk defines the codebook (kvcomp_encode.py:99-103)
            counts = kvcomp_cuda.symbol_counts([quant_ints])
            if self.codebook_smoothing:
                counts[:self._smoothed_symbols()] += 1
            codebook = self._host_codebook(counts)
        enc_table = self.encode_codebook if codebook is None else codebook[0].to(self.device)
        fn = kvcomp_cuda.k_entropy_encode_cuda_export if self.is_k else kvcomp_cuda.v_entropy_encode_cuda_export
        encoded_, block_infos_, vec_infos_ = fn(quant_ints, enc_table, bi_buf, ti_buf, idx_buf, payload_buf,
                                                self._encoded.used, self.head_num, self.head_dim)
        if codebook is not None:
            self._set_codebook(*codebook[:2], tree_format=codebook[2])
        self.max_tile_bytes = max(self.max_tile_bytes, kvcomp_cuda.last_encode_max_tile_bytes)
        self.max_stream_bytes = max(self.max_stream_bytes, kvcomp_cuda.last_encode_max_stream_bytes)
        self._append_encoded(encoded_)
        self._block_infos.append(block_infos_)
        self._thread_infos.append(vec_infos_)
        self._min_ints.append(min_ints)
        self._scales.append(quant_scale)
        self.compressed_ctx_len += quant_ints.shape[0] * quant_ints.shape[1]
        return quant_ints

    # The first chunk's codebook is built on the device (histogram, Huffman code, tables: no 256 reads of single counts
    # by the host and no wait before the encode is queued); False: by the host builder, as in the reference.
    device_codebook = True
    # With a codebook in place, store(want_symbols=False) queues the fused quantize + encode and returns without
    # waiting for it: sizes and errors are learnt the next time something asks for them (encoded_data, get_cr, ...),
    # and a store that fails on the device is reported by the next store() or attention call that finds its outcome
    # (poll_stores: no wait), or by whatever waits for sizes: the context is then rolled back to the last good store,
    # with the failed stores' tokens back in the tail.  The caches that models use switch it on, together with
    # codebook_smoothing, which rules out symbols without a code.
    async_store = False
    # stores of up to this many blocks are queued without a wait; longer ones (a second chunk of a prompt) are waited for
    ASYNC_KEEP_BLOCKS = 8

    def _encode_direct(self, T: int, *, tables, table_bytes, symbols=None, cache=None, mask=0, meta=None,
                       min_ints=None, quant_scale=None, keep=None, lost_if_dropped=False):
        """Queue one encode whose outputs go straight to their final places in this context's buffers; nothing waits.
        Quantizes `cache` on the fly (fused store) or takes `symbols` with their min_ints / quant_scale."""
        nb = T // self.block_size
        B, H, D = self.batch_size, self.head_num, self.head_dim
        sizes = kvcomp_cuda.buffer_sizes(T, B * H * D, self.is_k, H, D)
        gshape = mask_keepdim_shape((nb, self.block_size, B, H, D), dims_to_mask(self.quant_dims))
        state = self._device_state()
        if not self._unverified:
            self._sync_sizes()                                 # (a no-op unless sizes are outstanding for another reason)
            self._verified = self._bookkeeping() + (self._encoded.used,)
        bi = self._block_infos.reserve(sizes[0], (), torch.uint8, self.device)
        ti = self._thread_infos.reserve(sizes[1], (), torch.uint8, self.device)
        mn = self._min_ints.reserve(nb, gshape[1:], torch.int8, self.device)
        sc = self._scales.reserve(nb, gshape[1:], torch.float16, self.device)
        worst = T * B * H * D                                  # the reference's pre-allocation: a byte per symbol
        if (self._encoded.data is None or
                self._encoded.used + self._enc_pending + worst > self._encoded.data.numel()):
            self._sync_sizes()                                 # growing copies the filled part: it has to be known
            self._encoded.reserve(worst, (), torch.uint8, self.device)
        if cache is None:
            mn.copy_(min_ints)
            sc.copy_(quant_scale)
        kvcomp_cuda.encode_async(self.is_k, batch=B, head_num=H, head_dim=D, tokens=T, encode_tables=tables,
                                 table_bytes=table_bytes, block_infos=bi, thread_infos=ti, encoded=self._encoded.data,
                                 symbols=symbols, cache=cache, quant_mask=mask, eb=self.quant_scale_rel, min_ints=mn, scales=sc,
                                 codebook_meta=meta, stream_bytes=state[8:9], result=state[:8])
        self._block_infos.used += sizes[0]
        self._thread_infos.used += sizes[1]
        self._min_ints.used += nb
        self._scales.used += nb
        self._enc_pending += worst
        self.compressed_ctx_len += T
        self._unverified.append((T, keep, self._bookkeeping(), worst, lost_if_dropped))

    def _first_chunk_on_device(self, quant_ints, min_ints, quant_scale):
        """Codebook of the first stored chunk (kvcomp_encode.py:99-103) and its encode, queued back to back on the
        device: histogram -> Huffman code and tables (kvc_build_codebook_device) -> encode with the table where it lies.
        The host then reads the sizes (one wait) and keeps the codebook in the reference's form."""
        counts = kvcomp_cuda.symbol_counts_chunks(quant_ints.reshape(-1), 1)
        if self.codebook_smoothing:
            counts[0, :self._smoothed_symbols()] += 1
        T = quant_ints.shape[0] * quant_ints.shape[1]
        for fmt in (kvcomp_cuda.TREE_I8, kvcomp_cuda.TREE_I16):
            enc, trees, meta = kvcomp_cuda.build_codebook_device(counts, fmt)
            self._encode_direct(T, tables=enc, table_bytes=enc.shape[1], symbols=quant_ints, meta=meta, min_ints=min_ints,
                                quant_scale=quant_scale)
            self._trim_after_sync = True                       # a byte per symbol was reserved
            try:
                self._sync_sizes()                             # (a failure leaves the context as it was before the encode)
                break
            except KvcompError:
                # status 4: the code does not fit the int8 tree (kvc_build_codebook_device) -- once more with the wide one
                if fmt == kvcomp_cuda.TREE_I8 and int(meta[0, 3]) == 4:
                    continue
                raise
        shift, enc_bytes, dec_bytes, status = (int(v) for v in meta[0].cpu())
        assert status == 0 and shift == 0, "shift must be 0"
        self._set_codebook(enc[0, :enc_bytes].cpu(), trees[0, :dec_bytes].cpu(), tree_format=fmt)

    def _smoothed_symbols(self) -> int:
        return min(256, int(math.ceil(1.0 / self.quant_scale_rel)) + 3)      # symbols 0 .. ceil(1 / eb) + 2

    # The reference derives the one codebook of a stream from its first stored chunk alone, so a symbol that first
    # shows up later has no code (its encoder then emits nothing for it and the stream is corrupt; here the
    # encoder reports an error).  With smoothing, every symbol the error bound allows counts once more than it
    # occurs, so all of them get a code; the codebook then differs from the reference's for the same chunk.
    codebook_smoothing = False

    def _host_codebook(self, counts: torch.Tensor):
        """(encode table, decode tree, tree format) from 256 symbol counts, by the host builder: the reference's int8
        tree where the code fits it, the int16 tree where it does not (more than 64 symbols, or one above 127)."""
        try:
            shift, enc, dec = kvcomp_cuda.build_codebook_from_counts(counts, kvcomp_cuda.TREE_I8)
            fmt = kvcomp_cuda.TREE_I8
        except KvcompError:
            shift, enc, dec = kvcomp_cuda.build_codebook_from_counts(counts, kvcomp_cuda.TREE_I16)
            fmt = kvcomp_cuda.TREE_I16
        assert shift == 0, "shift must be 0"
        return enc, dec, fmt

    def _store_fused(self, to_compress: torch.Tensor, mask: int):
        """fp16 rows -> payload + metadata in one call (kvc_store_fused); same outputs as the two-step path."""
        T = to_compress.shape[0]
        nb = T // self.block_size
        gshape = mask_keepdim_shape((nb, self.block_size, self.batch_size, self.head_num, self.head_dim), mask)
        min_ints = torch.empty(gshape, dtype=torch.int8, device=self.device)
        quant_scale = torch.empty(gshape, dtype=torch.float16, device=self.device)
        sizes = kvcomp_cuda.buffer_sizes(T, self.batch_size * self.head_num * self.head_dim, self.is_k, self.head_num,
                                         self.head_dim)
        KVCompCtx.buffer_ctx_len[self.device] = T
        bi_buf, ti_buf, idx_buf, payload_buf = self._scratch(sizes)
        encoded_, block_infos_, vec_infos_ = kvcomp_cuda.store_fused(
            self.is_k, to_compress, mask, self.quant_scale_rel, self.encode_codebook, min_ints, quant_scale, bi_buf, ti_buf,
            idx_buf, payload_buf, self._encoded.used)
        self.max_tile_bytes = max(self.max_tile_bytes, kvcomp_cuda.last_encode_max_tile_bytes)
        self.max_stream_bytes = max(self.max_stream_bytes, kvcomp_cuda.last_encode_max_stream_bytes)
        self._append_encoded(encoded_)
        self._block_infos.append(block_infos_)
        self._thread_infos.append(vec_infos_)
        self._min_ints.append(min_ints)
        self._scales.append(quant_scale)
        self.compressed_ctx_len += T

    def _assert_ready(self):
        assert self.quant_min_ints is not None, "quant_min_ints is None"
        assert self.quant_scales is not None, "quant_scales is None"
        assert self.encoded_data is not None, "encoded_data is None"
        assert self.block_infos is not None, "huffman_block_info is None"
        assert self.thread_infos is not None, "huffman_thread_info is None"
        assert self.decode_codebook is not None, "decode_codebook is None"

    def get_decode_quant_ints(self) -> Tuple[torch.Tensor, float]:
        """kvcomp_encode.py:168-207: Huffman-decode the whole compressed part back to uint8 symbols."""
        self._assert_ready()
        decoded = torch.empty(self.compressed_ctx_len // self.block_size, self.block_size, self.batch_size,
                              self.head_num, self.head_dim, dtype=torch.uint8, device=self.device)
        fn = kvcomp_cuda.k_entropy_decode_cuda_export if self.is_k else kvcomp_cuda.v_entropy_decode_cuda_export
        t_ms = fn(self.encoded_data, self.block_infos, self.thread_infos, self.decode_codebook, decoded,
                  self.head_num, self.head_dim, self.tree_format)
        return decoded, t_ms

    # decode and dequantize in one kernel (no uint8 tensor in between); False = the reference's two steps
    fused_get = True

    def get_only_compressed(self) -> Tuple[torch.Tensor, float]:
        """kvcomp_encode.py:153-166: decode + dequantize the compressed part -> ([ctx_c, B, H, D] fp16, ms)."""
        if KVCompCtx.fused_get:
            self._assert_ready()
            out = torch.empty(self.compressed_ctx_len, self.batch_size, self.head_num, self.head_dim, dtype=torch.float16,
                              device=self.device)
            t_ms = kvcomp_cuda.decode_dequant(self.is_k, self.encoded_data, self.block_infos, self.thread_infos,
                                              self.decode_codebook, self.quant_min_ints, self.quant_scales,
                                              dims_to_mask(self.quant_dims), self.block_size, out, self.tree_format)
            return out, t_ms
        decoded, t_ms = self.get_decode_quant_ints()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        out = dequant(decoded, self.quant_min_ints, self.quant_scales, self.quant_dims)
        end.record()
        end.synchronize()
        return out.flatten(0, 1), t_ms + start.elapsed_time(end)

    def get(self) -> Tuple[torch.Tensor, float]:
        """kvcomp_encode.py:138-151: compressed part followed by the uncompressed tail.  (While nothing has
        been compressed yet the tail is everything; the reference asserts in that state.)"""
        if self.compressed_ctx_len == 0:
            return self.buffer.clone(), 0.0
        out, t_ms = self.get_only_compressed()
        if self.buffer is not None and self.buffer.shape[0] > 0:
            out = torch.cat([out, self.buffer], dim=0)
        return out, t_ms

    def mat_vec_mul(self, B: torch.Tensor) -> Tuple[torch.Tensor, float]:
        """kvcomp_encode.py:209-280.  K: B = q [B, H, D] -> scores [B, H, ctx_c].  V: B = p [B, H, ctx_c] ->
        [1, B, H, D] (the per-128-token partials summed, as the reference does in PyTorch)."""
        self._assert_ready()
        assert B.dtype == torch.float16, "B must be float16"
        assert len(B.shape) == 3, "B must be 3D tensor"
        assert B.shape[0] == self.batch_size, "batch size mismatch"
        assert B.shape[1] % self.head_num == 0, "head num mismatch"
        q_heads = B.shape[1]
        if self.is_k:
            assert B.shape[2] == self.head_dim, "head dim mismatch"
            C = torch.empty(self.batch_size, q_heads, self.compressed_ctx_len, dtype=torch.float16, device=self.device)
            t_ms = kvcomp_cuda.k_decode_and_mat_vec_mul_cuda_export(
                self.decode_codebook, self.block_infos, self.thread_infos, self.encoded_data,
                self.quant_min_ints.reshape(-1), self.quant_scales.reshape(-1), B.contiguous(), C, self.head_num, self.head_dim,
                self.tree_format)
            return C, t_ms
        assert B.shape[2] == self.compressed_ctx_len, "ctx len mismatch"
        C = torch.empty(self.compressed_ctx_len // kvcomp_cuda.V_VEC_LEN, self.batch_size, q_heads, self.head_dim,
                        dtype=torch.float16, device=self.device)
        t_ms = kvcomp_cuda.v_decode_and_mat_vec_mul_cuda_export(
            self.decode_codebook, self.block_infos, self.thread_infos, self.encoded_data,
            self.quant_min_ints.reshape(-1), self.quant_scales.reshape(-1), B.contiguous(), C, self.head_num, self.head_dim,
            self.tree_format)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        C = C.sum(dim=0, keepdim=True, dtype=torch.float32).to(torch.float16)
        end.record()
        end.synchronize()
        return C, t_ms + start.elapsed_time(end)

    def build_codebook(self, tensors: List[torch.Tensor]):
        """kvcomp_encode.py:282-306: one codebook from the quantized whole blocks of sample tensors."""
        assert len(tensors) > 0, "tensors must not be empty"
        device_ = tensors[0].device
        sym = []
        for cache in tensors:
            self._check(cache)
            assert device_ == cache.device, "device mismatch"
            blocked_len = cache.shape[0] // self.block_size * self.block_size
            blocked = cache[:blocked_len].reshape(-1, self.block_size, self.batch_size, self.head_num, self.head_dim)
            sym.append(quant(blocked, self.quant_dims, self.quant_scale_rel)[0])
        enc, dec, fmt = self._host_codebook(kvcomp_cuda.symbol_counts(sym))
        if self.device is None:
            self.device = device_
            KVCompCtx.buffer_ctx_len[self.device] = 0
        self._set_codebook(enc, dec, tree_format=fmt)

    def _set_codebook(self, enc: torch.Tensor, dec: torch.Tensor, tree_format: int = kvcomp_cuda.TREE_I8):
        """enc / dec: CPU byte tensors from kvcomp_cuda.build_codebook."""
        self.tree_format = tree_format
        lengths = enc.view(torch.int32)[1::2]
        self.max_code_bits = int(lengths.max())      # sizes the fused decoders' table in LDS
        self.encode_codebook = enc.to(self.device)
        self.decode_codebook = dec.to(self.device)

    @property
    def shape(self):
        return torch.Size([self.compressed_ctx_len, self.batch_size, self.head_num, self.head_dim])

    def held_bytes(self) -> int:
        """Device memory this context holds, from the capacities of its buffers (not just their filled parts)."""
        n = 0 if self._tail is None else self._tail.numel() * self._tail.element_size()
        for g in (self._encoded, self._block_infos, self._thread_infos, self._min_ints, self._scales):
            if g.data is not None:
                n += g.data.numel() * g.data.element_size()
        for t in (self.encode_codebook, self.decode_codebook):
            if t is not None:
                n += t.numel()
        return n

    def compressed_bytes(self) -> int:
        """Denominator of get_cr (kvcomp_encode.py:318-324): everything a fused kernel has to read."""
        return (self.block_infos.numel() + self.thread_infos.numel() + self.encoded_data.numel() +
                self.quant_min_ints.numel() + self.quant_scales.numel() * 2)

    def get_cr(self):
        """kvcomp_encode.py:317-326"""
        original = 2 * self.batch_size * self.compressed_ctx_len * self.head_num * self.head_dim
        return original / self.compressed_bytes()
