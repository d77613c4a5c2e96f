"""GPU tests of the compressed-cache context, modelled on the reference's own scripts: exact symbol round
trip after two appended stores (kvcomp_cuda_extension/scripts/test_py_ctx_k_2d_load.py:55-84, test_py_ctx_v.py),
repeated get (scripts/test_py_ctx_multiple_get.py:22-30), fused result against a dense matmul on the
dequantized cache (test_py_ctx_k_2d_load.py:129-134, here at 1e-3 instead of 1e-2), and prefill-then-append-one
(accuracy/reproduce_cuda_error.py:25-46)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _config(k_mode="BlockQuant", v_mode="TokenQuant", k_recent=64, v_recent=128, ebk=0.1, ebv=0.2):
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, QuantMode
    KVCompCacheConfigStatic.config = KVCompCacheConfig("synthetic", QuantMode(k_mode), QuantMode(v_mode), 64, 128,
                                                       k_recent, v_recent, ebk, ebv)


def _oracle_mask(ctx):
    from kvcomp_amd.compute import dims_to_mask
    return dims_to_mask(ctx.quant_dims)


@pytest.mark.parametrize("is_k,mode", [(True, "BlockQuant"), (True, "ChannelQuant"), (False, "TokenQuant"), (False, "VectorQuant")])
def test_twice_store_round_trip_and_get(is_k, mode):
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode=mode if is_k else "BlockQuant", v_mode=mode if not is_k else "TokenQuant")
    T, B, H, D = 1024, 1, 8, 128
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D)
    eb = 0.03 if is_k else 0.07                     # the reference scripts' error bounds
    ctx = KVCompCtx(is_k, B, H, D, eb)
    ctx.build_codebook([x.to(DEV), x.to(DEV)])
    q1 = ctx.store(x.to(DEV))
    q2 = ctx.store(x.to(DEV))
    assert ctx.ctx_len == 2 * T and ctx.compressed_ctx_len == 2 * T and ctx.buffer.shape[0] == 0
    quant_int = torch.cat([q1, q2], dim=0)
    decoded, ms = ctx.get_decode_quant_ints()
    assert torch.equal(decoded, quant_int)
    # symbols, min and scale equal the oracle's, store by store
    mask = _oracle_mask(ctx)
    o = O.quant(S.np16(S.blocked(x, ctx.block_size)), mask, eb)
    assert np.array_equal(q1.cpu().numpy(), o[3]) and np.array_equal(q2.cpu().numpy(), o[3])
    n = ctx.quant_scales.shape[0] // 2
    assert np.array_equal(ctx.quant_scales[:n].cpu().numpy().view(np.uint16), o[2].view(np.uint16))
    assert np.array_equal(ctx.quant_min_ints[n:].cpu().numpy(), o[4])
    # per-tile stream equals the oracle's encoder run with this context's codebook (second store: base offset)
    p1, bi1, ti1 = O.encode_tiles(o[3], is_k, ctx.encode_codebook.cpu().numpy(), 0)
    p2, bi2, ti2 = O.encode_tiles(o[3], is_k, ctx.encode_codebook.cpu().numpy(), p1.size)
    assert np.array_equal(ctx.encoded_data.cpu().numpy(), np.concatenate([p1, p2]))
    assert np.array_equal(ctx.block_infos.cpu().numpy(), np.concatenate([bi1, bi2]))
    assert np.array_equal(ctx.thread_infos.cpu().numpy(), np.concatenate([ti1, ti2]))
    # get(): bit-exact dequantized cache, idempotent
    full, _ = ctx.get()
    deq = O.dequant(o[3], o[4], o[2], mask).reshape(T, B, H, D)
    assert np.array_equal(full[:T].cpu().numpy().view(np.uint16), deq.view(np.uint16))
    assert np.array_equal(full[T:].cpu().numpy().view(np.uint16), deq.view(np.uint16))
    again, _ = ctx.get()
    assert torch.equal(full, again)
    # compression ratio formula (models/cache/kvcomp_encode.py:317-326)
    comp = (ctx.block_infos.numel() + ctx.thread_infos.numel() + ctx.encoded_data.numel() +
            ctx.quant_min_ints.numel() + 2 * ctx.quant_scales.numel())
    assert ctx.get_cr() == pytest.approx(2 * B * 2 * T * H * D / comp)
    assert tuple(ctx.shape) == (2 * T, B, H, D)


@pytest.mark.parametrize("is_k,mode", [(True, "BlockQuant"), (True, "ChannelQuant"), (False, "TokenQuant")])
def test_fused_mat_vec_mul_against_dense(is_k, mode):
    from kvcomp_amd.ctx import KVCompCtx
    import kvcomp_amd.kvcomp_cuda as m
    _config(k_mode=mode if is_k else "BlockQuant")
    T, B, H, D = 2048, 1, 8, 128
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D).to(DEV)
    ctx = KVCompCtx(is_k, B, H, D, 0.1 if is_k else 0.2)
    ctx.store(x)
    dense, _ = ctx.get_only_compressed()
    if is_k:
        q = S.synth_q(B, H, D).to(DEV)
        C, ms = ctx.mat_vec_mul(q)
        ref = torch.einsum("tbhd,bhd->bht", dense.float(), q.float())
        assert (C.float() - ref).abs().max() <= 1e-3 * ref.abs().max()
        base = torch.empty(T, B, H, dtype=torch.float16, device=DEV)
        m.k_mat_vec_mul_cuda_export(dense.contiguous(), q, base)         # the dense baseline on the same cache
        assert (base.float().permute(1, 2, 0) - ref).abs().max() <= 1e-3 * ref.abs().max()
    else:
        p = S.synth_p(B, H, T).to(DEV)
        C, ms = ctx.mat_vec_mul(p)
        ref = torch.einsum("tbhd,bht->bhd", dense.float(), p.float())
        assert tuple(C.shape) == (1, B, H, D)
        assert (C.float()[0] - ref).abs().max() <= 1e-3 * ref.abs().max()
    assert ms > 0


@pytest.mark.parametrize("D", [128, 96])
def test_fused_matvecs_with_subnormal_weights_in_some_heads(D):
    """In the default arithmetic the matrix-core kernels hand fp16 weights (q, or p without the softmax) to the matrix
    cores as the words they were loaded as, unless a weight of the tile is subnormal: then the tile's weights are split
    into a high part (zero where subnormal) and a low part scaled into the normal range.  Heads alternate here between
    ordinary and entirely subnormal weights, so a wave that works through several tiles switches between the two
    forms: every head's result must match the dense product (a head whose low parts were lost would come out zero),
    and runs of three tiles must give the bits of single tiles."""
    from kvcomp_amd import _lib
    from kvcomp_amd import attention as A
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant")
    T, B, H = 640, 2, 6
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(S.synth_k(T, B, H, D).to(DEV))
    vctx.store(S.synth_v(T, B, H, D).to(DEV))
    assert 1 <= kctx.max_code_bits <= 7 and 1 <= vctx.max_code_bits <= 7      # the matrix-core kernels' range
    q, p = S.synth_q(B, H, D).to(DEV), S.synth_p(B, H, T).to(DEV).clamp_min(2e-4)      # (no subnormal p in the even heads)
    for w in (q, p):                                       # odd heads: a few 1e-5, below fp16's smallest normal 6.1e-5
        small = w[:, 1::2].float()
        w[:, 1::2] = (small / small.abs().max() * 5e-5).to(torch.float16)
        assert (w[:, 1::2].float().abs() < 6.1e-5).all() and (w[:, 1::2] != 0).any()
    for ctx, w, fn in ((kctx, q, A.k_scores), (vctx, p, A.v_partials)):
        lut = A.build_lut(ctx.decode_codebook, ctx.tree_format)
        out = {}
        for tpw in (1, 3):
            was = _lib.set_option("fused_tiles_per_wave", tpw)
            try:
                out[tpw] = fn(ctx, lut, w)[0]
            finally:
                _lib.set_option("fused_tiles_per_wave", was)
        assert torch.equal(out[1], out[3])
        dense = ctx.get_only_compressed()[0].float()
        if ctx.is_k:
            got, ref = out[1], torch.einsum("tbhd,bhd->bht", dense, w.float())
        else:
            got, ref = out[1].sum(dim=0), torch.einsum("tbhd,bht->bhd", dense, w.float())
        err, scale = (got - ref).abs().amax(dim=2), ref.abs().amax(dim=2)
        assert (scale > 0).all() and (err <= 1e-3 * scale).all(), (err / scale).max()


def test_prefill_then_append_one_token_at_a_time():
    from kvcomp_amd.ctx import KVCompCtx
    _config(v_recent=256)
    T0, extra, B, H, D = 952, 300, 1, 4, 128
    x = S.synth_v(T0 + extra, B, H, D).to(DEV)
    ctx = KVCompCtx(False, B, H, D, 0.04)
    ctx.store(x[:T0].contiguous())
    for i in range(T0, T0 + extra):
        ctx.store(x[i:i + 1].contiguous())
        if i % 50 == 0:
            full, _ = ctx.get()
            assert full.shape[0] == i + 1
    full, _ = ctx.get()
    assert ctx.ctx_len == T0 + extra and full.shape[0] == T0 + extra
    c = ctx.compressed_ctx_len
    assert c % 128 == 0 and 128 <= ctx.ctx_len - c < 256 + 128 and ctx.buffer.shape[0] == ctx.ctx_len - c
    assert torch.equal(full[c:], x[c:])                                # the tail is stored verbatim
    # the compressed part: per-token quantization does not depend on how the tokens were chunked
    o = O.quant(S.np16(S.blocked(x[:c].cpu(), 128)), O.MASK_V_TOKEN, 0.04)
    deq = O.dequant(o[3], o[4], o[2], O.MASK_V_TOKEN).reshape(c, B, H, D)
    assert np.array_equal(full[:c].cpu().numpy().view(np.uint16), deq.view(np.uint16))
    assert np.array_equal(ctx.get_decode_quant_ints()[0].cpu().numpy(), o[3])


def test_a_context_holds_little_more_than_its_stream():
    """After a long prompt the fp16 tail is a few blocks, not the prompt: device memory held (capacities, not just
    the filled parts) stays well below the dense cache, and a failed store leaves the context unchanged."""
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd._lib import KvcompError
    _config(k_mode="ChannelQuant")
    T, B, H, D = 4096, 2, 4, 128
    for is_k in (True, False):
        x = (S.synth_k if is_k else S.synth_v)(T + 17, B, H, D).to(DEV)
        ctx = KVCompCtx(is_k, B, H, D, 0.1 if is_k else 0.2)
        ctx.store(x[:T], want_symbols=False)
        for i in range(T, T + 17):
            ctx.store(x[i:i + 1], want_symbols=False)
        dense = 2 * (T + 17) * B * H * D
        assert ctx._tail.shape[0] <= 2 * (ctx.block_size + ctx.recent_size) + 64
        assert ctx.held_bytes() <= 0.45 * dense, (ctx.held_bytes(), dense)
        assert ctx.held_bytes() >= ctx.compressed_bytes() + ctx.buffer.numel() * 2
        full, _ = ctx.get()
        assert torch.equal(full[ctx.compressed_ctx_len:], x[ctx.compressed_ctx_len:])
    # a store whose encode fails (a symbol the codebook has no code for) changes nothing
    _config(k_mode="BlockQuant")
    ctx = KVCompCtx(True, 1, 2, 128, 0.1)
    flat = torch.zeros(128, 1, 2, 128, dtype=torch.float16, device=DEV)
    flat[::2] = 1.0                                               # two symbols only: 0 and 10
    ctx.store(flat)
    before = (ctx.ctx_len, ctx.compressed_ctx_len, ctx.buffer.shape[0], ctx.encoded_data.numel())
    wide = S.synth_k(128, 1, 2, 128).to(DEV)                      # needs the symbols in between
    with pytest.raises(KvcompError):
        ctx.store(wide)
    assert before == (ctx.ctx_len, ctx.compressed_ctx_len, ctx.buffer.shape[0], ctx.encoded_data.numel())
    ctx.store(flat)                                               # and the context still works
    assert ctx.ctx_len == 256


def test_batch_and_gqa_heads():
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant")
    T, B, H, D, rep = 512, 2, 2, 128, 4
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    s, _ = kctx.mat_vec_mul(q)
    kd, _ = kctx.get_only_compressed()
    ref = torch.einsum("tbhd,bhd->bht", kd.float().repeat_interleave(rep, dim=2), q.float())
    assert (s.float() - ref).abs().max() <= 1e-3 * ref.abs().max()
    p = torch.softmax(s.float() / D ** 0.5, dim=-1).half()
    o, _ = vctx.mat_vec_mul(p)
    vd, _ = vctx.get_only_compressed()
    ref = torch.einsum("tbhd,bht->bhd", vd.float().repeat_interleave(rep, dim=2), p.float())
    assert (o.float()[0] - ref).abs().max() <= 1e-3 * ref.abs().max()


def test_smoke_entry():
    import __graft_entry__ as g
    g.smoke()


@pytest.mark.parametrize("k_mode,rep,extra", [("ChannelQuant", 1, 0), ("ChannelQuant", 4, 37), ("BlockQuant", 2, 200)])
def test_compressed_attention_matches_fp32_reference(k_mode, rep, extra, fused_mode):
    """Full decode attention (scores -> 1/sqrt(d) -> softmax -> p.V, grouped-query heads, uncompressed tails)
    against fp32 PyTorch attention over the dequantized cache: 1e-3 relative to max|out|."""
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode=k_mode)
    T, B, H, D = 1024 + extra, 2, 2, 128
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    out = CompressedAttention(kctx, vctx).attend(q)
    kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
    assert kd.shape[0] == T and vd.shape[0] == T
    s = torch.einsum("tbhd,bhd->bht", kd.repeat_interleave(rep, dim=2), q.float()) / D ** 0.5
    ref = torch.einsum("tbhd,bht->bhd", vd.repeat_interleave(rep, dim=2), torch.softmax(s, dim=-1))
    assert (out - ref).abs().max() <= 1e-3 * ref.abs().max()
    # element by element: within 1e-3 of the value itself, or of the output's typical size for the smallest ones
    if fused_mode.rounded:
        assert torch.allclose(out, ref, rtol=1e-3, atol=1e-3 * float(ref.pow(2).mean().sqrt()))


@pytest.mark.parametrize("rows", [0, 1])
@pytest.mark.parametrize("tiles_per_wave", [1, 2, 3])
@pytest.mark.parametrize("D", [128, 96])
def test_compressed_attention_under_every_staging_plan(rows, tiles_per_wave, D, fused_mode):
    """The fused kernels may decode from the packed payload or from per-lane rows, and a wave may take one
    tile or a run of tiles (fetching one ahead): every combination must give the same attention output,
    including runs that are cut short at the end of a tile row (3 does not divide the tile columns)."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant")
    T, B, H, rep = 512 + 19, 2, 4, 2
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    assert 0 < kctx.max_stream_bytes <= kctx.max_tile_bytes and 0 < kctx.max_code_bits <= 32
    q = S.synth_q(B, H * rep, D).to(DEV)
    L = _lib.lib()
    default_plan = CompressedAttention(kctx, vctx).attend(q)
    was_rows, was_tiles = _lib.set_option("fused_rows", rows), _lib.set_option("fused_tiles_per_wave", tiles_per_wave)
    try:
        out = CompressedAttention(kctx, vctx).attend(q)
    finally:
        _lib.set_option("fused_rows", was_rows)
        _lib.set_option("fused_tiles_per_wave", was_tiles)
    kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
    s = torch.einsum("tbhd,bhd->bht", kd.repeat_interleave(rep, dim=2), q.float()) / D ** 0.5
    ref = torch.einsum("tbhd,bht->bhd", vd.repeat_interleave(rep, dim=2), torch.softmax(s, dim=-1))
    # the plan changes where the bits are read from, not the arithmetic: results are identical, except that per-lane
    # rows are only implemented by the fp32-FMA kernels, whose sums are rounded in a different order than the
    # matrix cores' (both carry the products exactly)
    same_kernel = (rows == 1) == (was_rows == 1) or fused_mode.mfma == 0      # (was_rows: what the environment preset)
    if same_kernel:
        assert torch.equal(out, default_plan)
    else:
        assert (out - default_plan).abs().max() <= 1e-5 * default_plan.abs().max()
    assert (out - ref).abs().max() <= fused_mode.tol_vs_fp16_cache * ref.abs().max()
    assert L.kvc_set_option(b"no_such_option", 1) != 0


@pytest.mark.parametrize("schedule", [46030, 85035, 25040, 30000, 166020, 10000])
@pytest.mark.parametrize("D,rep", [(128, 1), (96, 2)])
def test_compressed_attention_under_every_tile_schedule(schedule, D, rep):
    """The matrix-core kernels of a long stream walk the row-major tile sequence in segments, the waves of a segment
    taking runs of 8, 4, 2 or 1 consecutive tiles (across tile rows, and cut short where a segment or the stream ends).
    Forced here on a small cache whose tile counts are no multiple of any run: every schedule must give the output of
    the plain launch bit for bit, in both arithmetic modes."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant")
    T, B, H = 7 * 128 + 31, 2, 3                      # K: 14 x 6 tiles; V: 7 rows of 12 (D 128) or 9 (D 96) tiles
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    for rounded in (1, 0):
        saved = {n: _lib.set_option(n, v_) for n, v_ in (("fused_rounded", rounded), ("fused_schedule", 0))}
        try:
            plain = CompressedAttention(kctx, vctx).attend(q)
            _lib.set_option("fused_schedule", schedule)
            out = CompressedAttention(kctx, vctx).attend(q)
        finally:
            for n, v_ in saved.items():
                _lib.set_option(n, v_)
        assert torch.equal(out, plain)
    kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
    s_ = torch.einsum("tbhd,bhd->bht", kd.repeat_interleave(rep, dim=2), q.float()) / D ** 0.5
    ref = torch.einsum("tbhd,bht->bhd", vd.repeat_interleave(rep, dim=2), torch.softmax(s_, dim=-1))
    assert (plain - ref).abs().max() <= 3e-3 * ref.abs().max()          # (the unrounded mode's result was the last)


@pytest.mark.parametrize("D,rep,eb_k", [(128, 1, 0.1), (96, 2, 0.05), (64, 4, 0.3), (128, 8, 0.1)])
def test_lane_permute_in_assembly_equals_the_compilers(D, rep, eb_k):
    """The fp32-FMA kernels fetch one of four operands from the lanes of a quad with a permute that rides on the
    multiply-add (inline assembly, which the compiler's hazard handling cannot see into).  The same kernels with
    the permute expressed through the compiler's intrinsic must give the same bits, for the one-symbol loops (K)
    and the two-symbol loop (V), skewed and plain staging, one and two tiles per wave."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant", ebk=eb_k)
    T, B, H = 1024 + 13, 2, 2
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, eb_k), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    saved = {n: _lib.set_option(n, v_) for n, v_ in (("fused_rounded", 0), ("fused_mfma", 0))}
    try:
        for skew in (0, 1):
            for tpw in (1, 2):
                _lib.set_option("fused_skew", skew)
                _lib.set_option("fused_tiles_per_wave", tpw)
                _lib.set_option("fused_builtin_dpp", 0)
                asm = CompressedAttention(kctx, vctx).attend(q)
                _lib.set_option("fused_builtin_dpp", 1)
                builtin = CompressedAttention(kctx, vctx).attend(q)
                assert torch.isfinite(asm).all() and torch.equal(asm, builtin), (skew, tpw)
    finally:
        for n, v_ in saved.items():
            _lib.set_option(n, v_)
        _lib.set_option("fused_skew", -1)
        _lib.set_option("fused_tiles_per_wave", 0)
        _lib.set_option("fused_builtin_dpp", 0)


@pytest.mark.parametrize("hint", ["too_small", "absent"])
def test_compressed_attention_with_wrong_or_missing_size_hints(hint, fused_mode):
    """The encoder's size hints only size the LDS staging: with hints that are too small (tiles do not fit and
    are decoded from global memory) or absent the result must not change."""
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant")
    T, B, H, D, rep = 256, 1, 2, 128, 1
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    good = CompressedAttention(kctx, vctx).attend(q)
    for c in (kctx, vctx):
        if hint == "too_small":
            c.max_tile_bytes, c.max_stream_bytes, c.max_code_bits = 16, 4, 1
        else:
            c.max_tile_bytes = c.max_stream_bytes = c.max_code_bits = 0
    again = CompressedAttention(kctx, vctx).attend(q)
    assert (again - good).abs().max() <= 1e-5 * good.abs().max()


@pytest.mark.parametrize("T,D,rep,B", [(40, 128, 1, 1), (100, 128, 2, 2), (300, 64, 4, 1), (531, 96, 2, 2), (1024, 128, 8, 1)])
def test_one_call_attention_matches_stepwise_and_fp32(T, D, rep, B, fused_mode):
    """kvc_attention_decode (scores, per-group softmax, weighted values and the final merge inside the library)
    against the same result assembled step by step with PyTorch's softmax, and against fp32 attention over the
    dequantized cache.  Covers: nothing compressed yet, K compressed but V not, tails of different lengths."""
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant")
    H = 2
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    q = S.synth_q(B, H * rep, D).to(DEV)
    att = CompressedAttention(kctx, vctx)
    ms = []
    out = att.attend(q, kernel_ms=ms)
    assert len(ms) == 2 and (ms[0] > 0) == (kctx.compressed_ctx_len > 0) and (ms[1] > 0) == (vctx.compressed_ctx_len > 0)
    again = att.attend(q)                                   # workspace reuse, no timing
    assert torch.equal(out, again)
    step = att.attend_stepwise(q)
    # the stepwise path rounds the softmax weights to fp16 (the reference kernel's input format)
    assert (out - step).abs().max() <= 2e-3 * step.abs().max()
    kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
    s = torch.einsum("tbhd,bhd->bht", kd.repeat_interleave(rep, dim=2), q.float()) / D ** 0.5
    ref = torch.einsum("tbhd,bht->bhd", vd.repeat_interleave(rep, dim=2), torch.softmax(s, dim=-1))
    assert (out - ref).abs().max() <= fused_mode.tol_vs_fp16_cache * ref.abs().max()


def test_one_call_attention_grows_with_the_cache(fused_mode):
    """Prefill, then decode steps that push blocks out of the tails: attention after every few steps stays
    within tolerance of fp32 attention over what get() returns."""
    from kvcomp_amd.ctx import KVCompCtx
    from kvcomp_amd.attention import CompressedAttention
    _config(k_mode="ChannelQuant")
    B, H, D, rep = 1, 4, 128, 2
    T0, steps = 200, 140
    k, v = S.synth_k(T0 + steps, B, H, D).to(DEV), S.synth_v(T0 + steps, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k[:T0])
    vctx.store(v[:T0])
    att = CompressedAttention(kctx, vctx)
    q = S.synth_q(B, H * rep, D).to(DEV)
    for i in range(steps):
        kctx.store(k[T0 + i:T0 + i + 1])
        vctx.store(v[T0 + i:T0 + i + 1])
        if i % 23 == 0 or i == steps - 1:
            out = att.attend(q)
            kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
            s = torch.einsum("tbhd,bhd->bht", kd.repeat_interleave(rep, dim=2), q.float()) / D ** 0.5
            ref = torch.einsum("tbhd,bht->bhd", vd.repeat_interleave(rep, dim=2), torch.softmax(s, dim=-1))
            assert (out - ref).abs().max() <= fused_mode.tol_vs_fp16_cache * ref.abs().max(), "step %d" % i


@pytest.mark.parametrize("device_codebook", [True, False])
def test_a_fine_error_bound_falls_back_to_the_wide_tree(device_codebook):
    """More than 64 symbols do not fit the reference's int8 decode tree (include/huffman.h:18-22): the context then
    keeps a 5-byte-node tree and tells every decoder, instead of failing the store and every store after it."""
    from kvcomp_amd import container, kvcomp_cuda
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.compute import dequant
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant")
    T, B, H, D = 512, 1, 2, 128
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.004), KVCompCtx(False, B, H, D, 0.2)
    kctx.device_codebook = device_codebook
    sym = kctx.store(k)
    vctx.store(v)
    assert int(sym.max()) > 127 and kctx.tree_format == kvcomp_cuda.TREE_I16 and vctx.tree_format == kvcomp_cuda.TREE_I8
    assert kctx.decode_codebook.numel() % 5 == 0
    # the host builder's wide tree for the same counts, byte for byte
    _, enc, dec = kvcomp_cuda.build_codebook([sym], kvcomp_cuda.TREE_I16)
    assert torch.equal(kctx.encode_codebook.cpu(), enc) and torch.equal(kctx.decode_codebook.cpu(), dec)
    dec_sym, _ = kctx.get_decode_quant_ints()
    assert torch.equal(dec_sym, sym)
    full, _ = kctx.get_only_compressed()
    ref = dequant(sym, kctx.quant_min_ints, kctx.quant_scales, kctx.quant_dims).flatten(0, 1)
    assert torch.equal(full.view(torch.int16), ref.view(torch.int16))
    again = kctx.store(k)                                    # a second store with the codebook in place
    assert torch.equal(again, sym) and kctx.compressed_ctx_len == 2 * T
    vctx.store(v)
    q = S.synth_q(B, H, D).to(DEV)
    out = CompressedAttention(kctx, vctx).attend(q)
    kd, vd = kctx.get()[0].float(), vctx.get()[0].float()
    s = torch.einsum("tbhd,bhd->bht", kd, q.float()) / D ** 0.5
    want = torch.einsum("tbhd,bht->bhd", vd, torch.softmax(s, dim=-1))
    assert (out - want).abs().max() <= 1e-3 * want.abs().max()
    assert torch.equal(kctx.mat_vec_mul(q)[0].float(), kctx.mat_vec_mul(q)[0].float())
    scores = kctx.mat_vec_mul(q)[0].float()
    dense = torch.einsum("tbhd,bhd->bht", kd, q.float())
    assert (scores - dense).abs().max() <= 2e-3 * dense.abs().max()       # fp16 scores out
    # the container carries the node format
    back = container.loads(container.dumps(kctx), DEV)
    assert back.tree_format == kvcomp_cuda.TREE_I16
    assert torch.equal(back.get_only_compressed()[0], kctx.get_only_compressed()[0])


@pytest.mark.parametrize("is_k,mode,B,H,D", [(True, "ChannelQuant", 2, 3, 96), (True, "BlockQuant", 1, 4, 128),
                                              (False, "TokenQuant", 2, 3, 96), (False, "VectorQuant", 2, 4, 128)])
def test_one_kernel_get_equals_decode_then_dequant(is_k, mode, B, H, D):
    """kvc_decode_dequant against the reference's two steps (kvcomp_encode.py:153-166) and against the oracle."""
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode=mode if is_k else "BlockQuant", v_mode=mode if not is_k else "TokenQuant")
    T = 512
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D)
    ctx = KVCompCtx(is_k, B, H, D, 0.1)
    ctx.store(x.to(DEV))
    assert ctx.compressed_ctx_len == T
    try:
        KVCompCtx.fused_get = True
        one, _ = ctx.get_only_compressed()
        KVCompCtx.fused_get = False
        two, _ = ctx.get_only_compressed()
    finally:
        KVCompCtx.fused_get = True
    assert one.shape == two.shape == (T, B, H, D)
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    mask = _oracle_mask(ctx)
    o = O.quant(S.np16(S.blocked(x, ctx.block_size)), mask, 0.1)
    deq = O.dequant(o[3], o[4], o[2], mask).reshape(T, B, H, D)
    assert np.array_equal(one.cpu().numpy().view(np.uint16), deq.view(np.uint16))


def test_attention_call_can_be_captured_in_a_graph(fused_mode):
    """kvc_attention_decode allocates nothing and waits for nothing, so a serving loop can record it in a HIP graph.
    The graph is replayed several times with eager work and synchronisations of the program's own in between, for
    queries that change between replays (the graph reads q and writes out in place), with and without fp16 tails;
    every replay must equal the eager call bit for bit."""
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    B, H, Hq, D = 2, 2, 8, 128
    for T in (512, 512 + 37):
        k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
        kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
        kctx.store(k)
        vctx.store(v)
        attn = CompressedAttention(kctx, vctx)
        q = S.synth_q(B, Hq, D).to(DEV)
        out = torch.empty(B, Hq, D, dtype=torch.float32, device=DEV)
        attn.attend(q, out=out)                                   # builds the tables and the workspace
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                attn.attend(q, out=out)
        torch.cuda.synchronize()
        g = torch.Generator(device=DEV).manual_seed(4)
        for i in range(4):
            q.copy_(torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.float16))
            eager = attn.attend(q).clone()                        # eager work between the replays
            torch.cuda.synchronize()
            out.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), (T, i)
