"""The benchmark configurations at their full sizes, checked through properties that need no CPU oracle run:
decode(encode(quantize(x))) returns the quantizer's symbols exactly, the fused store produces the same stream
as quantize-then-encode, decode + dequantize equals the dequantized symbols bit for bit and stays inside the
error bound, and decode attention on the compressed cache matches fp32 PyTorch attention over the dequantized
cache within 1e-3 of max|reference|.  Inputs are the synthetic distributions of the benchmark (the seeded host
generators of tests/_synth.py, as bench.py uses them); the long-context configuration runs at each of its three K
error bounds."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CONFIGS = {
    # batch, kv heads, q heads, head_dim, tokens, eb K, eb V, distribution
    "cfg2": (1, 32, 32, 128, 4096, 0.1, 0.2, "gauss"),
    "cfg3": (16, 8, 32, 128, 8192, 0.1, 0.2, "gauss"),
    "cfg5": (4, 32, 32, 96, 32768, 0.1, 0.3, "laplace"),
    "cfg5_eb_k_0.05": (4, 32, 32, 96, 32768, 0.05, 0.3, "laplace"),
    "cfg5_eb_k_0.2": (4, 32, 32, 96, 32768, 0.2, 0.3, "laplace"),
}


def _make(name):
    import bench
    B, H, Hq, D, T, ebk, ebv, dist = CONFIGS[name]
    cfg = dict(B=B, H=H, Hq=Hq, D=D, T=T, eb_k=ebk, eb_v=ebv, dist=dist)
    return bench.make_kv(cfg, torch.device(DEV))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size_round_trip_and_attention(name):
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.compute import QuantMode, dequant, quant
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, KVCompCtx
    B, H, Hq, D, T, ebk, ebv, _ = CONFIGS[name]
    KVCompCacheConfigStatic.config = KVCompCacheConfig(name, QuantMode.ChannelQuant, QuantMode.TokenQuant, 64, 128, 64, 128, ebk, ebv)
    k, v = _make(name)
    ctxs = []
    for is_k, x, eb in ((True, k, ebk), (False, v, ebv)):
        ctx = KVCompCtx(is_k, B, H, D, eb)
        sym = ctx.store(x)                                             # first store: symbol path, builds the codebook
        assert ctx.compressed_ctx_len == T and sym.numel() == x.numel()
        # decode(encode(.)) is the identity on the symbols
        dec, _ = ctx.get_decode_quant_ints()
        assert torch.equal(dec, sym)
        # the fused store yields the same stream
        twin = KVCompCtx(is_k, B, H, D, eb)
        twin.device = ctx.device
        twin._set_codebook(ctx.encode_codebook.cpu(), ctx.decode_codebook.cpu())
        assert twin.store(x, want_symbols=False) is None
        for attr in ("encoded_data", "block_infos", "thread_infos", "quant_min_ints", "quant_scales"):
            assert torch.equal(getattr(twin, attr), getattr(ctx, attr)), attr
        del twin
        # decode + dequantize == dequantized symbols, and within the error bound of the input
        full, _ = ctx.get_only_compressed()
        ref = dequant(sym, ctx.quant_min_ints, ctx.quant_scales, ctx.quant_dims).flatten(0, 1)
        assert torch.equal(full.view(torch.int16), ref.view(torch.int16))
        gshape = ctx.quant_scales.shape
        bound = 0.53 * ctx.quant_scales.float()                        # src/compute.cpp:60-69
        err = (full.float() - x.float()).abs().reshape(-1, ctx.block_size, B, H, D)
        assert bool((err <= bound.expand(err.shape) + 1e-3 * x.float().abs().reshape(err.shape)).all()), gshape
        del sym, dec, full, ref, err
        ctxs.append(ctx)
    kctx, vctx = ctxs
    assert kctx.get_cr() > 2.5 and vctx.get_cr() > 4.0
    g = torch.Generator(device=DEV).manual_seed(1236)
    q = torch.randn(B, Hq, D, generator=g, device=DEV, dtype=torch.float32).to(torch.float16)
    from kvcomp_amd import _lib
    was = _lib.set_option("fused_rounded", 0)
    try:
        out = CompressedAttention(kctx, vctx).attend(q)
        out_r = None
        _lib.set_option("fused_rounded", 1)
        out_r = CompressedAttention(kctx, vctx).attend(q)              # matrix-core kernels
        was_m = _lib.set_option("fused_mfma", 0)
        out_rf = CompressedAttention(kctx, vctx).attend(q)             # the same arithmetic on the fp32-FMA kernels
        _lib.set_option("fused_mfma", was_m)
    finally:
        _lib.set_option("fused_rounded", was)
    rep = Hq // H
    qd = q.double().reshape(B, H, rep, D)

    def attention(kd, vd):                                              # [T, B, H, D] float64 -> [B, Hq, D]
        s = torch.einsum("tbhd,bhrd->bhrt", kd, qd) / math.sqrt(D)
        return torch.einsum("bhrt,tbhd->bhrd", torch.softmax(s, dim=-1), vd).reshape(B, Hq, D)

    # (1) The fused kernels multiply q by (sym + min) * scale as it stands, in fp32.  Against attention over
    #     that exact dequantization they agree to fp32 accuracy.
    exact = []
    for ctx in (kctx, vctx):
        sym, _ = ctx.get_decode_quant_ints()
        exact.append(((sym.double() + ctx.quant_min_ints.double()) * ctx.quant_scales.double()).flatten(0, 1))
        del sym
    ref_exact = attention(*exact)
    del exact
    scale = float(ref_exact.abs().max())
    assert float((out.double() - ref_exact).abs().max()) <= 1e-4 * scale
    # (2) The reference's dequantizer rounds every value to fp16 (models/cache/kvcomp_encode.py:146).  Attention
    #     over that fp16 cache differs from (1) by the cache's own rounding noise, which the x20 outlier channels
    #     of the synthetic K amplify through the softmax: that noise, not the kernels, sets the distance
    #     below (1e-3 of max|reference| on the heavy-tailed data, a few 1e-3 on the outlier-channel data).
    ref_fp16 = attention(kctx.get()[0].double(), vctx.get()[0].double())
    noise = float((ref_fp16 - ref_exact).abs().max())
    dist = float((out.double() - ref_fp16).abs().max())
    assert abs(dist - noise) <= 0.05 * noise + 1e-4 * scale            # the whole distance is that rounding noise
    assert dist <= 2e-2 * scale
    # (3) In rounded mode the kernels round each dequantized value to fp16 first, like that dequantizer: then they
    #     meet the fp16-cache reference itself within 1e-3 of max|reference|.
    assert float((out_r.double() - ref_fp16).abs().max()) <= 1e-3 * scale
    assert float((out_rf.double() - ref_fp16).abs().max()) <= 1e-3 * scale
    # ... element by element too: within 1e-3 of the value, or of the output's typical size for the smallest ones
    assert torch.allclose(out_r.double(), ref_fp16, rtol=1e-3, atol=1e-3 * float(ref_fp16.pow(2).mean().sqrt()))


def test_cfg4_layer_at_its_own_shape_through_the_append_loop():
    """One layer of the full-decode configuration at its own shape: batch 8, 32 heads x 128, a 4096-token prompt and
    130 appended tokens through KVCompCtx as the model-facing caches set it up (stores queued without a wait, codebook
    smoothing), K recompressing every 64 and V every 128 tokens.  After tokens 1, 64, 65, 128, 129 and 130 the
    attention operator (compressed part + fp16 tails) must match float64 attention over get() within 1e-3, and the
    queued stores must have produced the stream of a context that waits for every store.  Reference contract:
    models/cache/kvcomp_encode.py:345-360 (update), models/llama.py:279-304 (attention over what update returns)."""
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.compute import QuantMode
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, KVCompCtx
    B, H, D, T, NEW = 8, 32, 128, 4096, 130
    KVCompCacheConfigStatic.config = KVCompCacheConfig("cfg4", QuantMode.ChannelQuant, QuantMode.TokenQuant, 64, 128, 64, 128, 0.1, 0.2)
    import bench
    cfg = dict(B=B, H=H, Hq=H, D=D, T=T + 192, eb_k=0.1, eb_v=0.2, dist="gauss")
    k, v = bench.make_kv(cfg, torch.device(DEV))
    g = torch.Generator(device=DEV).manual_seed(1236)
    ctxs = {}
    for name, asynchronous in (("queued", True), ("waiting", False)):
        kc, vc = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
        for c in (kc, vc):
            c.codebook_smoothing = True
            c.async_store = asynchronous
        kc.store(k[:T], want_symbols=False)
        vc.store(v[:T], want_symbols=False)
        ctxs[name] = (kc, vc)
    kc, vc = ctxs["queued"]
    attn = CompressedAttention(kc, vc)

    def check(step):
        q = torch.randn(B, H, D, generator=g, device=DEV, dtype=torch.float32).to(torch.float16)
        out = attn.attend(q)
        kd, vd = kc.get()[0], vc.get()[0]                               # [T, B, H, D] fp16: compressed part + tail
        assert kd.shape[0] == vd.shape[0] == T + step
        worst = 0.0
        for b in range(B):                                              # a batch entry at a time keeps float64 small
            s = torch.einsum("thd,hd->ht", kd[:, b].double(), q[b].double()) / math.sqrt(D)
            ref = torch.einsum("ht,thd->hd", torch.softmax(s, dim=-1), vd[:, b].double())
            scale = float(ref.abs().max())
            worst = max(worst, float((out[b].double() - ref).abs().max()) / scale)
            assert torch.allclose(out[b].double(), ref, rtol=1e-3, atol=1e-3 * float(ref.pow(2).mean().sqrt()))
        assert worst <= 1e-3, (step, worst)
        return worst

    # (1e-3 against the fp16 cache is the statement about the default arithmetic, whatever the environment presets)
    from kvcomp_amd import _lib
    was = _lib.set_option("fused_rounded", 1)
    try:
        check(0)
        seen = set()
        for i in range(NEW):
            for name in ("queued", "waiting"):
                ctxs[name][0].store(k[T + i:T + i + 1], want_symbols=False)
                ctxs[name][1].store(v[T + i:T + i + 1], want_symbols=False)
            if i + 1 in (1, 64, 65, 128, 129, 130):
                check(i + 1)
                seen.add((kc.compressed_ctx_len, vc.compressed_ctx_len))
    finally:
        _lib.set_option("fused_rounded", was)
    assert len(seen) >= 3                                               # the checks saw K and V recompress
    assert kc.waits == 1 and vc.waits == 1                              # nothing since the prompt's codebook has waited
    for a, b in zip(ctxs["queued"], ctxs["waiting"]):
        assert a.compressed_ctx_len == b.compressed_ctx_len > T - 128 and a.ctx_len == b.ctx_len == T + NEW
        for name in ("encoded_data", "block_infos", "thread_infos", "quant_min_ints", "quant_scales", "buffer"):
            assert torch.equal(getattr(a, name), getattr(b, name)), name
