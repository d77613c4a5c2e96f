"""Fused quantize + encode (kvc_store_fused) against the oracle and against the two-step path: group
parameters, thread_infos, block_infos and payload must be byte-identical, for every supported layout,
batch > 1, head_dim 96 and 128, Gaussian and heavy-tailed data, and appended stores (base offset)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S
from tests.test_gpu_ctx import _config, _oracle_mask

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CASES = [  # is_k, mode, B, H, D, dist
    (True, "ChannelQuant", 1, 4, 128, "gauss"),
    (True, "ChannelQuant", 2, 3, 96, "laplace"),
    (True, "BlockQuant", 1, 4, 128, "gauss"),
    (True, "BlockQuant", 2, 2, 64, "gauss"),
    (False, "TokenQuant", 1, 4, 128, "gauss"),
    (False, "TokenQuant", 2, 4, 96, "laplace"),
    (False, "TokenQuant", 3, 2, 32, "gauss"),
    # magnitudes far from 1: the packed fp16 quantizer rescales every group by a power of two
    (True, "ChannelQuant", 1, 2, 128, "gauss_tiny"),
    (True, "ChannelQuant", 2, 2, 96, "laplace_big"),
    (True, "BlockQuant", 1, 2, 64, "gauss_big"),
    (False, "TokenQuant", 2, 2, 96, "laplace_tiny"),
    (False, "TokenQuant", 1, 4, 128, "gauss_big"),
]


def _data(is_k, T, B, H, D, dist, seed):
    dist, _, mag = dist.partition("_")
    # exact power-of-two factors: group scales near 2^-12 (small normal and subnormal fp16 values) and near 2^7
    factor = {"": 1.0, "tiny": 2.0 ** -12, "big": 2.0 ** 6}[mag]
    if dist == "laplace":
        x = S.synth_laplace(T, B, H, D, seed)
    else:
        x = (S.synth_k if is_k else S.synth_v)(T, B, H, D, seed)
    return x if factor == 1.0 else (x.float() * factor).clamp(-60000.0, 60000.0).to(torch.float16)


@pytest.mark.parametrize("is_k,mode,B,H,D,dist", CASES)
def test_fused_store_equals_oracle_and_two_step_path(is_k, mode, B, H, D, dist):
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode=mode if is_k else "BlockQuant", v_mode=mode if not is_k else "TokenQuant", k_recent=64, v_recent=128)
    T = 512
    eb = 0.1 if is_k else 0.2
    x1, x2 = _data(is_k, T, B, H, D, dist, 11), _data(is_k, T, B, H, D, dist, 12)
    fused, plain = KVCompCtx(is_k, B, H, D, eb), KVCompCtx(is_k, B, H, D, eb)
    for ctx in (fused, plain):
        ctx.build_codebook([x1.to(DEV), x2.to(DEV)])
    assert fused.store(x1.to(DEV), want_symbols=False) is None           # codebook known: the fused path runs
    assert fused.store(x2.to(DEV), want_symbols=False) is None
    q1 = plain.store(x1.to(DEV))
    q2 = plain.store(x2.to(DEV))
    assert q1 is not None and q2 is not None
    assert fused.compressed_ctx_len == plain.compressed_ctx_len == 2 * T
    for name in ("quant_scales", "quant_min_ints", "thread_infos", "block_infos", "encoded_data"):
        a, b = getattr(fused, name), getattr(plain, name)
        assert a.shape == b.shape and a.dtype == b.dtype, name
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.uint8 else a, b.view(torch.uint8) if b.dtype != torch.uint8 else b), name
    assert (fused.max_tile_bytes, fused.max_stream_bytes) == (plain.max_tile_bytes, plain.max_stream_bytes)
    # and against the oracle, store by store
    mask = _oracle_mask(fused)
    table = fused.encode_codebook.cpu().numpy()
    off, payloads, bis, tis, scales, mins = 0, [], [], [], [], []
    for x in (x1, x2):
        o = O.quant(S.np16(S.blocked(x, fused.block_size)), mask, eb)
        p, bi, ti = O.encode_tiles(o[3], is_k, table, off, vec_len=D if is_k else 128)
        off += p.size
        payloads.append(p); bis.append(bi); tis.append(ti); scales.append(o[2].ravel()); mins.append(o[4].ravel())
    assert np.array_equal(fused.encoded_data.cpu().numpy(), np.concatenate(payloads))
    assert np.array_equal(fused.block_infos.cpu().numpy(), np.concatenate(bis))
    assert np.array_equal(fused.thread_infos.cpu().numpy(), np.concatenate(tis))
    assert np.array_equal(fused.quant_scales.cpu().numpy().ravel().view(np.uint16), np.concatenate(scales).view(np.uint16))
    assert np.array_equal(fused.quant_min_ints.cpu().numpy().ravel(), np.concatenate(mins))
    # the decoder reads it back
    dec, _ = fused.get_decode_quant_ints()
    assert torch.equal(dec, torch.cat([q1, q2], dim=0))


def test_fused_store_in_the_append_loop_matches_the_symbol_path():
    """Prefill, then one token at a time (accuracy/reproduce_cuda_error.py:25-46): the cache built through the
    fused store equals the one built through the symbol path at every recompression."""
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    T0, steps, B, H, D = 952, 200, 2, 2, 128
    for is_k in (True, False):
        x = _data(is_k, T0 + steps, B, H, D, "gauss", 5).to(DEV)
        a, b = KVCompCtx(is_k, B, H, D, 0.1), KVCompCtx(is_k, B, H, D, 0.1)
        a.store(x[:T0].contiguous(), want_symbols=False)         # first store builds the codebook (symbol path)
        b.store(x[:T0].contiguous())
        for i in range(T0, T0 + steps):
            a.store(x[i:i + 1].contiguous(), want_symbols=False)
            b.store(x[i:i + 1].contiguous())
        assert a.compressed_ctx_len == b.compressed_ctx_len > T0 - 128
        assert torch.equal(a.encoded_data, b.encoded_data) and torch.equal(a.thread_infos, b.thread_infos)
        assert torch.equal(a.block_infos, b.block_infos)
        assert torch.equal(a.get()[0], b.get()[0])


def test_unsupported_layout_uses_the_symbol_path():
    from kvcomp_amd import kvcomp_cuda
    from kvcomp_amd.compute import dims_to_mask
    assert not kvcomp_cuda.store_fused_supported(False, dims_to_mask([4]), 1, 4, 128)      # VectorQuant
    assert not kvcomp_cuda.store_fused_supported(True, dims_to_mask([2, 3, 4]), 1, 4, 128)
    assert kvcomp_cuda.store_fused_supported(True, dims_to_mask([1]), 2, 4, 96)


@pytest.mark.parametrize("B,H,D", [(2, 4, 128), (3, 2, 96), (1, 2, 32)])
def test_fused_store_per_token_and_batch_groups(B, H, D):
    """V with one scale / minimum per (token, batch entry) (group dimensions [3, 4], mask 0xC): the layout the fused
    store accepts besides the ones KVCompCtx uses; called directly, compared with the oracle byte for byte."""
    from kvcomp_amd import kvcomp_cuda as m
    T, eb, mask = 256, 0.2, O.MASK_SIM_TOKEN
    assert m.store_fused_supported(False, mask, B, H, D)
    x = _data(False, T, B, H, D, "gauss", 31)
    x5 = S.np16(S.blocked(x, 64))
    _, _, scale, sym, mn = O.quant(x5, mask, eb)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts)
    _, enc = O.encode_table(code, length, counts)
    payload, bi, ti = O.encode_tiles(sym.reshape(T // 128, 128, B, H, D), False, enc, 0, vec_len=128)
    sizes = m.buffer_sizes(T, B * H * D, False, H, D)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    g_min = torch.zeros(scale.size, dtype=torch.int8, device=DEV)
    g_scale = torch.zeros(scale.size, dtype=torch.float16, device=DEV)
    g_enc, g_bi, g_ti = m.store_fused(False, x.to(DEV).contiguous(), mask, eb, torch.from_numpy(enc).to(DEV), g_min, g_scale,
                                      bufs[0], bufs[1], bufs[2], bufs[3], 0)
    assert np.array_equal(g_scale.cpu().numpy().view(np.uint16), scale.ravel().view(np.uint16))
    assert np.array_equal(g_min.cpu().numpy(), mn.ravel())
    assert np.array_equal(g_ti.cpu().numpy(), ti) and np.array_equal(g_bi.cpu().numpy(), bi)
    assert np.array_equal(g_enc.cpu().numpy(), payload)


def _pair_of_contexts(T0, extra, B, H, D, k_mode="ChannelQuant"):
    """The same tokens stored into a context that waits for every encode and into one that does not."""
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, KVCompCtx, QuantMode
    KVCompCacheConfigStatic.config = KVCompCacheConfig("synthetic", QuantMode(k_mode), QuantMode("TokenQuant"), 64, 128,
                                                       64, 128, 0.1, 0.2)
    out = []
    for is_k in (True, False):
        x = (S.synth_k if is_k else S.synth_v)(T0 + extra, B, H, D).to(DEV)
        pair = []
        for asynchronous in (False, True):
            ctx = KVCompCtx(is_k, B, H, D, 0.1 if is_k else 0.2)
            ctx.codebook_smoothing = True
            ctx.async_store = asynchronous
            ctx.store(x[:T0], want_symbols=False)
            for i in range(T0, T0 + extra):
                ctx.store(x[i:i + 1], want_symbols=False)
            pair.append(ctx)
        out.append(pair)
    return out


@pytest.mark.parametrize("k_mode", ["ChannelQuant", "BlockQuant"])
def test_store_without_waiting_gives_the_same_stream(k_mode):
    """async_store queues the fused quantize + encode of every block that leaves the tail, writes its outputs straight
    to their final places and never asks the device for a size; the stream must equal the waiting path's byte for
    byte (payload, metadata, quantization parameters, size hints), and attention over it must not need the sizes."""
    from kvcomp_amd.attention import CompressedAttention
    B, H, D = 2, 2, 128
    (k_sync, k_async), (v_sync, v_async) = _pair_of_contexts(300, 400, B, H, D, k_mode)
    q = S.synth_q(B, 2 * H, D).to(DEV)
    assert k_async.waits == 1 and v_async.waits == 1                       # the first chunk's codebook; no store since has waited
    out_async = CompressedAttention(k_async, v_async).attend(q)            # an address and a bound are enough
    assert k_async.waits == 1 and v_async.waits == 1
    out_sync = CompressedAttention(k_sync, v_sync).attend(q)
    assert torch.equal(out_async, out_sync)
    for a, b in ((k_sync, k_async), (v_sync, v_async)):
        assert a.compressed_ctx_len == b.compressed_ctx_len > 300 and a.ctx_len == b.ctx_len == 700
        for name in ("encoded_data", "block_infos", "thread_infos", "quant_min_ints", "quant_scales", "buffer"):
            assert torch.equal(getattr(a, name), getattr(b, name)), name
        assert b._enc_pending == 0                                          # reading encoded_data learnt the sizes
        assert (a.max_tile_bytes, a.max_stream_bytes) == (b.max_tile_bytes, b.max_stream_bytes)
        assert a.get_cr() == b.get_cr()
        assert torch.equal(a.get()[0], b.get()[0])


def test_append_and_attend_can_be_captured_in_a_graph():
    """One decode step of a layer -- append a block of tokens to K and V (quantize + encode, outputs in place) and
    attend over everything -- recorded in a HIP graph: the step allocates nothing, waits for nothing and records no
    memset.  The graph first puts the two device counters back where they stood, so that every replay appends at the
    same place; each replay (with eager work in between) must equal the eager step bit for bit."""
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, KVCompCtx, QuantMode
    KVCompCacheConfigStatic.config = KVCompCacheConfig("synthetic", QuantMode.ChannelQuant, QuantMode.TokenQuant, 64, 128,
                                                       64, 128, 0.1, 0.2)
    B, H, Hq, D, T0, NEW = 2, 2, 4, 128, 512, 128
    k, v = S.synth_k(T0 + NEW, B, H, D).to(DEV), S.synth_v(T0 + NEW, B, H, D).to(DEV)
    q = S.synth_q(B, Hq, D).to(DEV)

    def fresh():
        kc, vc = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
        for c, x in ((kc, k), (vc, v)):
            c.codebook_smoothing = True
            c.async_store = True
            c.store(x[:T0], want_symbols=False)
        return kc, vc

    kc, vc = fresh()
    att = CompressedAttention(kc, vc)
    kc.store(k[T0:], want_symbols=False)
    vc.store(v[T0:], want_symbols=False)
    eager = att.attend(q).clone()
    torch.cuda.synchronize()

    kc, vc = fresh()
    att = CompressedAttention(kc, vc)
    out = torch.empty(B, Hq, D, dtype=torch.float32, device=DEV)
    att.attend(q, out=out)                                   # decode tables and workspace exist before the capture
    # one eager step makes every buffer as large as the step needs; then the host's view is put back
    for c in (kc, vc):
        c._sync_sizes()                                       # nothing outstanding: the host's view is exact
    saved = [(c._device_state().clone(), c._encoded.used, c._block_infos.used, c._thread_infos.used, c._min_ints.used,
              c._scales.used, c.compressed_ctx_len, c.ctx_len, c._tail_len, c._enc_pending) for c in (kc, vc)]
    kc.store(k[T0:], want_symbols=False)
    vc.store(v[T0:], want_symbols=False)
    att.attend(q, out=out)
    torch.cuda.synchronize()

    def rewind():
        for c, sv in zip((kc, vc), saved):
            c._state.copy_(sv[0])
            (c._encoded.used, c._block_infos.used, c._thread_infos.used, c._min_ints.used, c._scales.used,
             c.compressed_ctx_len, c.ctx_len, c._tail_len, c._enc_pending) = sv[1:]
            c._unverified, c._probe = [], None

    def step():
        rewind()
        kc.store(k[T0:], want_symbols=False)
        vc.store(v[T0:], want_symbols=False)
        att.attend(q, out=out)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for i in range(3):
        out.fill_(float("nan"))
        scratch = torch.randn(1 << 20, device=DEV).sum()     # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), i
    assert kc.encoded_data.numel() > 0 and float(scratch) == float(scratch)


def test_unbuilt_codebook_flags_the_encode_on_the_device():
    """A codebook that kvc_build_codebook_device could not build (a block with one symbol only) makes the batched
    encode fail when its result is read, not silently produce a stream."""
    import kvcomp_amd.kvcomp_cuda as m
    from kvcomp_amd._lib import KvcompError
    T, B, H, D = 128, 1, 2, 128
    sym = torch.randint(0, 9, (2, 64, B, H, D), dtype=torch.uint8, device=DEV)
    sym[1] = 3                                               # the second block holds a single symbol
    counts = m.symbol_counts_chunks(sym, 2)
    enc, trees, meta = m.build_codebook_device(counts)
    assert meta[:, 3].tolist() == [0, 1]
    sizes = m.calculate_buffer_size(sym, True, H, D)
    bi, ti = (torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes[:2])
    payload = torch.zeros(sizes[3], dtype=torch.uint8, device=DEV)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    m.encode_async(True, batch=B, head_num=H, head_dim=D, tokens=T, symbols=sym, encode_tables=enc, table_bytes=enc.shape[1],
                   table_stride=enc.shape[1], rows_per_codebook=1, codebook_meta=meta, block_infos=bi, thread_infos=ti,
                   encoded=payload, result=result)
    with pytest.raises(KvcompError, match="codebook"):
        m.encode_result(result, payload.numel())


@pytest.mark.parametrize("one_pass", [0, 2, 3])
@pytest.mark.parametrize("is_k,D,dist", [(True, 96, "laplace"), (False, 128, "gauss"), (True, 128, "gauss_tiny")])
def test_one_pass_and_two_pass_encoders_write_the_same_bytes(is_k, D, dist, one_pass):
    """The tile encoder runs in one pass (waves look back over the sizes published by the tiles before them; one or
    two tiles per wave) or in two (count, offsets, emit): payload, block_infos and thread_infos must not depend on
    which, for the fused store and for the encoder that starts from symbols, over enough tiles (> 4096) that waves of
    many workgroups wait for each other, and for a second store appended behind the first."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    T, B, H = 4096, 2, 16
    eb = 0.1 if is_k else 0.2
    x1, x2 = _data(is_k, T, B, H, D, dist, 21).to(DEV), _data(is_k, 512, B, H, D, dist, 22).to(DEV)
    results = []
    for mode in (1, one_pass):                       # the default first, then the variant under test
        was = _lib.set_option("encode_one_pass", mode)
        try:
            fused, plain = KVCompCtx(is_k, B, H, D, eb), KVCompCtx(is_k, B, H, D, eb)
            for ctx in (fused, plain):
                ctx.build_codebook([x1[:512], x2])
            fused.store(x1, want_symbols=False)
            fused.store(x2, want_symbols=False)
            plain.store(x1)
            plain.store(x2)
            results.append((fused, plain))
        finally:
            _lib.set_option("encode_one_pass", was)
    (f1, p1), (f2, p2) = results
    for name in ("quant_scales", "quant_min_ints", "thread_infos", "block_infos", "encoded_data"):
        a = getattr(f1, name)
        for other in (p1, f2, p2):
            b = getattr(other, name)
            assert a.shape == b.shape and torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name
    assert (f1.max_tile_bytes, f1.max_stream_bytes) == (f2.max_tile_bytes, f2.max_stream_bytes) == (p2.max_tile_bytes, p2.max_stream_bytes)
    # and the oracle agrees with the first store's payload
    o = O.quant(S.np16(S.blocked(x1.cpu(), f1.block_size)), _oracle_mask(f1), eb)
    pay, bi, ti = O.encode_tiles(o[3], is_k, f1.encode_codebook.cpu().numpy(), 0, vec_len=D if is_k else 128)
    assert np.array_equal(f1.encoded_data.cpu().numpy()[:pay.size], pay)
    assert np.array_equal(f1.block_infos.cpu().numpy()[:bi.size], bi)


@pytest.mark.parametrize("from_symbols", [False, True])
@pytest.mark.parametrize("is_k,T,B,H,D", [(True, 64 * 7, 1, 9, 96), (True, 64 * 19, 3, 1, 128), (False, 128 * 21, 1, 2, 96),
                                          (False, 128 * 57, 1, 1, 64), (True, 64 * 3, 3, 7, 72), (True, 64 * 9, 1, 7, 40)])
def test_one_pass_runs_of_two_over_odd_tile_counts(is_k, T, B, H, D, from_symbols):
    """Two tiles per wave forced on streams of 63 and 57 tiles: the last wave holds a single tile, which also
    closes the last (short) group of tiles; the first group is a full one of 56.  From fp16 and from uint8 symbols
    (which the one-pass kernel fetches through its LDS tile: head sizes whose words do not divide the 64 lanes
    included).  Payload and metadata must be the oracle's, and a second store must continue behind the first."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    eb = 0.1 if is_k else 0.2
    x = _data(is_k, T, B, H, D, "gauss", 31).to(DEV)
    was = _lib.set_option("encode_one_pass", 3)
    try:
        ctx = KVCompCtx(is_k, B, H, D, eb)
        ctx.build_codebook([x])
        ctx.store(x, want_symbols=from_symbols)
        ctx.store(x, want_symbols=from_symbols)
    finally:
        _lib.set_option("encode_one_pass", was)
    o = O.quant(S.np16(S.blocked(x.cpu(), ctx.block_size)), _oracle_mask(ctx), eb)
    pay, bi, ti = O.encode_tiles(o[3], is_k, ctx.encode_codebook.cpu().numpy(), 0, vec_len=D if is_k else 128)
    assert bi.size // 8 in (57, 63)
    got_bi, got_ti, got = ctx.block_infos.cpu().numpy(), ctx.thread_infos.cpu().numpy(), ctx.encoded_data.cpu().numpy()
    assert np.array_equal(got_bi[:bi.size], bi) and np.array_equal(got_ti[:ti.size], ti)
    assert np.array_equal(got[:pay.size], pay) and np.array_equal(got[pay.size:2 * pay.size], pay)
    second = got_bi[bi.size:2 * bi.size].view(np.uint32).reshape(-1, 2)
    first = bi.view(np.uint32).reshape(-1, 2)
    assert np.array_equal(second[:, 0], first[:, 0] + pay.size) and np.array_equal(second[:, 1], first[:, 1])


def test_a_queued_store_that_fails_is_reported_without_a_wait_and_taken_back():
    """async_store with codebook smoothing off: a block that needs a symbol the first chunk's codebook has no code for
    fails on the device, after store() has returned.  The next store() or attention call that finds the outcome (no
    wait) raises, and the context is then what it was after the last good store: bookkeeping, device words and
    payload position rolled back, the failed block's tokens back in front of the tail, nothing lost."""
    from kvcomp_amd._lib import KvcompError
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="BlockQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    B, H, D = 1, 2, 128
    flat = torch.zeros(256, B, H, D, dtype=torch.float16, device=DEV)
    flat[::2] = 1.0                                               # two symbols only: 0 and 10
    wide = S.synth_k(64, B, H, D).to(DEV)                         # needs the symbols in between
    ctx = KVCompCtx(True, B, H, D, 0.1)
    ctx.async_store = True
    ctx.store(flat, want_symbols=False)                           # first chunk: codebook of two symbols
    ctx.store(flat[:64], want_symbols=False)                      # a good block, queued
    torch.cuda.synchronize()
    ctx.poll_stores()                                             # its outcome has arrived: known to be good, no wait
    assert ctx.waits == 1 and not ctx._unverified and ctx.compressed_ctx_len == 320
    good = (ctx.compressed_ctx_len, ctx.block_infos.numel(), ctx.thread_infos.numel(), ctx.quant_scales.numel(),
            ctx.encoded_data.numel(), ctx.max_tile_bytes)
    payload = ctx.encoded_data.clone()
    ctx.store(wide, want_symbols=False)                           # fails on the device; store() cannot know yet
    assert ctx.compressed_ctx_len == 384
    one = torch.full((1, B, H, D), 0.5, dtype=torch.float16, device=DEV)
    taken = 0
    with pytest.raises(KvcompError, match="no code"):
        for _ in range(3):                                        # the outcome arrives some microseconds later
            ctx.store(one, want_symbols=False)                    # finds it, if it is there, before it does anything else
            taken += 1
            torch.cuda.synchronize()
    assert taken <= 1 and ctx.waits == 2                          # (the one wait that fetched the library's message)
    assert good == (ctx.compressed_ctx_len, ctx.block_infos.numel(), ctx.thread_infos.numel(), ctx.quant_scales.numel(),
                    ctx.encoded_data.numel(), ctx.max_tile_bytes)
    assert torch.equal(ctx.encoded_data, payload)
    assert ctx.ctx_len == 384 + taken and ctx.buffer.shape[0] == 64 + taken      # the store that raised took nothing in
    assert torch.equal(ctx.buffer[:64], wide) and torch.equal(ctx.buffer[64:], one[:taken])
    assert ctx._state[:5].tolist() == [ctx._state[0].item(), 0, 0, 0, ctx.block_infos.numel() // 8] and int(ctx._state[8]) == payload.numel()
    full, _ = ctx.get()
    assert torch.equal(full[:320], torch.cat([flat, flat[:64]])) and torch.equal(full[320:], ctx.buffer)
    # the block that cannot be encoded is still in the tail, so the next store that reaches a block boundary fails the same way
    with pytest.raises(KvcompError, match="no code"):
        for _ in range(200):
            ctx.store(one, want_symbols=False)
            torch.cuda.synchronize()
    assert ctx.compressed_ctx_len == 320 and torch.equal(ctx.encoded_data, payload)


def test_a_second_prompt_chunk_leaves_no_worst_case_reservation_behind():
    """A long store into a context that has its codebook reserves a byte per symbol for the payload; the reservation
    is given back once the sizes are known, so the context holds little more than its stream."""
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    T, B, H, D = 4096, 2, 4, 128
    for is_k in (True, False):
        x = (S.synth_k if is_k else S.synth_v)(2 * T, B, H, D).to(DEV)
        ctx = KVCompCtx(is_k, B, H, D, 0.1 if is_k else 0.2)
        ctx.codebook_smoothing = True
        ctx.async_store = True
        ctx.store(x[:T], want_symbols=False)
        ctx.store(x[T:], want_symbols=False)                      # waited for: longer than ASYNC_KEEP_BLOCKS blocks
        assert ctx.compressed_ctx_len >= 2 * T - 128 and not ctx._unverified
        tail_bytes = ctx._tail.numel() * 2
        assert ctx.held_bytes() - tail_bytes <= 1.5 * ctx.compressed_bytes(), (ctx.held_bytes(), ctx.compressed_bytes())
        twin = KVCompCtx(is_k, B, H, D, 0.1 if is_k else 0.2)
        twin.codebook_smoothing = True
        twin.store(x[:T], want_symbols=False)
        twin.store(x[T:], want_symbols=False)
        assert torch.equal(ctx.encoded_data, twin.encoded_data) and torch.equal(ctx.block_infos, twin.block_infos)


def test_size_hints_follow_queued_stores_without_a_wait():
    """The largest tile and the longest stream (which size the fused decoders' LDS areas) are brought up to date from
    the copies of the device words that arrive behind queued stores: no wait, and no stale hints over a long decode."""
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    B, H, D = 2, 2, 128
    quiet = (S.synth_k(256, B, H, D) * 0.0 + S.synth_k(256, B, H, D, 5).sign()).to(torch.float16).to(DEV)   # two levels per channel
    busy = S.synth_k(256, B, H, D, 6).to(DEV)
    a, b = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(True, B, H, D, 0.1)
    for c in (a, b):
        c.codebook_smoothing = True
    a.async_store = True
    for c in (a, b):
        c.store(quiet, want_symbols=False)                        # small tiles first
        for i in range(256):
            c.store(busy[i:i + 1], want_symbols=False)            # larger ones later
    torch.cuda.synchronize()
    a.poll_stores()
    assert a.waits == 1
    assert (a.max_tile_bytes, a.max_stream_bytes) == (b.max_tile_bytes, b.max_stream_bytes)
    assert a.max_tile_bytes > 0 and a._enc_pending == 0
