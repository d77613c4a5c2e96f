"""The model-facing cache classes (KVCompCachePytorchQuant / KVCompCache / KVCompCacheCuda): update() and
get_seq_length() against a CPU restatement of the reference's sim path made of stock PyTorch fp16 tensor ops."""
import math

import pytest
import torch

from tests import _synth as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# utils/compute.py:138-143: reduced dimensions of the [B, H, NB, BS, D] view
SIM_DIMS = {"BlockQuant": [1, 3, 4], "ChannelQuant": [3], "TokenQuant": [1, 4], "VectorQuant": [4]}


def _set_config(k_mode, v_mode, k_bs=64, v_bs=64, k_recent=64, v_recent=64, ebk=0.1, ebv=0.2, enable_quant=True,
                pre_rope=False):
    from kvcomp_amd.compute import QuantMode
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic
    KVCompCacheConfigStatic.extract_cache = None
    KVCompCacheConfigStatic.config = KVCompCacheConfig("test", QuantMode(k_mode), QuantMode(v_mode), k_bs, v_bs, k_recent,
                                                       v_recent, ebk, ebv, enable_quant=enable_quant,
                                                       enable_pre_rope=pre_rope)
    return KVCompCacheConfigStatic.config


def _sim_cpu(x_bhtd, block_size, eb, mode):
    """quant_ints + (quant_int + min_quant) * quant_scale (utils/compute.py:74-91,124-131) with PyTorch's own
    CPU fp16 ops -- library routines, op for op what the reference executes."""
    x = x_bhtd.cpu()
    B, H, T, D = x.shape
    t = x.reshape(B, H, -1, block_size, D)
    mn, mx = t, t
    for d in SIM_DIMS[mode]:
        mn = mn.min(dim=d, keepdim=True).values
        mx = mx.max(dim=d, keepdim=True).values
    scale = (mx - mn) * eb
    min_q = (mn / scale).round()
    q = (t / scale).round() - min_q
    return ((q + min_q) * scale).reshape(B, H, T, D)


def _expected(history, block_size, recent, eb, mode, steps):
    """Replays the tail bookkeeping of quant_error / cut_tensor (utils/compute.py:44-57,108-133) on the CPU."""
    done, total = 0, 0
    out = history.cpu().clone()
    for n_new in steps:
        total += n_new
        tail = total - done
        n = (tail + block_size - tail % block_size - recent) // block_size
        if n > 0:
            out[:, :, done:done + n * block_size] = _sim_cpu(history[:, :, done:done + n * block_size], block_size, eb, mode)
            done += n * block_size
    return out[:, :, :total], done


def _rope(T, D):
    pos = torch.arange(T, dtype=torch.float32)
    inv = 1.0 / (10000 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(pos, inv)
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos()[None].to(torch.float16), emb.sin()[None].to(torch.float16)        # [1, T, D]


@pytest.mark.parametrize("mode", ["BlockQuant", "ChannelQuant", "TokenQuant", "VectorQuant"])
def test_quant_dequant_sim_is_bit_exact(mode):
    from kvcomp_amd.compute import QuantMode, quant_dequant_sim
    B, H, T, D = 2, 3, 256, 96
    x = S.synth_k(T, B, H, D).permute(1, 2, 0, 3).contiguous()       # [B, H, T, D]
    got = quant_dequant_sim(x.to(DEV), 64, 0.1, QuantMode(mode)).cpu()
    ref = _sim_cpu(x, 64, 0.1, mode)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("mode,offset", [("ChannelQuant", 40.0), ("TokenQuant", 40.0), ("ChannelQuant", 12.0), ("TokenQuant", 12.0)])
def test_quant_dequant_sim_keeps_minima_outside_int8(mode, offset):
    """Groups that sit far from zero relative to their range have min/scale beyond +-127 (about 800 and 240 here); the
    sim path keeps them as fp16 numbers (the entropy-coded path would wrap them into int8).  Quotients beyond +-512
    are also outside what the two-elements-per-instruction quantizer covers: those groups take the fp32 chain, the
    ones at 240 the packed arithmetic (rows of 512 elements and 64-token blocks are kept in registers either way)."""
    from kvcomp_amd.compute import QuantMode, quant_dequant_sim
    g = torch.Generator().manual_seed(5)
    x = (torch.rand(1, 8, 128, 64, generator=g) * 0.5 + offset).to(torch.float16)
    got = quant_dequant_sim(x.to(DEV), 64, 0.1, QuantMode(mode)).cpu()
    ref = _sim_cpu(x, 64, 0.1, mode)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    assert (got.float() - x.float()).abs().max() < 0.1


@pytest.mark.parametrize("k_mode,v_mode,pre_rope", [("ChannelQuant", "TokenQuant", False), ("BlockQuant", "VectorQuant", False),
                                                    ("ChannelQuant", "TokenQuant", True)])
def test_update_prefill_then_decode_matches_cpu_replay(k_mode, v_mode, pre_rope):
    """accuracy/reproduce_cuda_error.py:25-46 in spirit: a prefill that is not a multiple of the block, then one
    token at a time across several block boundaries; every returned (K, V) equals the CPU replay bit for bit."""
    from kvcomp_amd.cache import KVCompCache
    from kvcomp_amd.compute import apply_rotary_pos_emb_single
    cfg = _set_config(k_mode, v_mode, k_recent=64, v_recent=128, pre_rope=pre_rope)
    B, H, D, L = 2, 4, 64, 2
    steps = [150] + [1] * 140
    T = sum(steps)
    ks = [S.synth_k(T, B, H, D, seed=11 + l).permute(1, 2, 0, 3).contiguous() for l in range(L)]
    vs = [S.synth_v(T, B, H, D, seed=21 + l).permute(1, 2, 0, 3).contiguous() for l in range(L)]
    cos, sin = _rope(T, D)
    cache = KVCompCache(B, H, D, L)
    assert cache.get_seq_length(0) == 0
    pos = 0
    for i, n_new in enumerate(steps):
        kw = {"cos": cos[:, pos:pos + n_new].to(DEV), "sin": sin[:, pos:pos + n_new].to(DEV)}
        for l in range(L):
            K, V = cache.update(ks[l][:, :, pos:pos + n_new].to(DEV), vs[l][:, :, pos:pos + n_new].to(DEV), l, kw)
        pos += n_new
        assert cache.get_seq_length(L - 1) == pos and K.shape == (B, H, pos, D) and V.shape == (B, H, pos, D)
        if i in (0, 1, 42, 43, 106, 107, len(steps) - 1):          # around the boundaries and at the end
            l = L - 1
            k_in = ks[l][:, :, :pos]
            if not pre_rope:
                k_in = torch.cat([apply_rotary_pos_emb_single(ks[l][:, :, a:b], cos[:, a:b], sin[:, a:b])
                                  for a, b in _chunks(steps[:i + 1])], dim=2)
            ek, k_done = _expected(k_in, cfg.k_block_size, cfg.k_recent_size, cfg.k_quant_scale_rel, k_mode, steps[:i + 1])
            ev, v_done = _expected(vs[l][:, :, :pos], cfg.v_block_size, cfg.v_recent_size, cfg.v_quant_scale_rel, v_mode, steps[:i + 1])
            if pre_rope:
                ek = apply_rotary_pos_emb_single(ek, cos[:, :pos], sin[:, :pos])
            assert torch.equal(K.cpu().view(torch.int16), ek.view(torch.int16)), "K differs at step %d" % i
            assert torch.equal(V.cpu().view(torch.int16), ev.view(torch.int16)), "V differs at step %d" % i
            inst = cache.cache_instance
            assert (inst.compressed_k_cache[l].shape[2] if inst.compressed_k_cache[l] is not None else 0) == k_done
            assert inst.k_cache_buffer[l].shape[2] == pos - k_done
            assert (inst.compressed_v_cache[l].shape[2] if inst.compressed_v_cache[l] is not None else 0) == v_done


def _chunks(steps):
    a = 0
    for n in steps:
        yield a, a + n
        a += n


def test_update_disabled_quant_keeps_raw_history_and_collects():
    from kvcomp_amd.cache import JumpOutException, KVCompCachePytorchQuant
    from kvcomp_amd.ctx import ExtractCacheConfig, KVCompCacheConfigStatic
    _set_config("ChannelQuant", "TokenQuant", enable_quant=False)
    B, H, D = 1, 2, 64
    k = S.synth_k(70, B, H, D).permute(1, 2, 0, 3).contiguous().to(DEV)
    v = S.synth_v(70, B, H, D).permute(1, 2, 0, 3).contiguous().to(DEV)
    cos, sin = _rope(70, D)
    zero = {"cos": torch.ones_like(cos).to(DEV), "sin": torch.zeros_like(sin).to(DEV)}       # identity rotation
    c = KVCompCachePytorchQuant(B, H, D, 2)
    KVCompCacheConfigStatic.extract_cache = ExtractCacheConfig(collect_round=KVCompCachePytorchQuant.round_)
    try:
        K, V = c.update(k[:, :, :69], v[:, :, :69], 1, {"cos": zero["cos"][:, :69], "sin": zero["sin"][:, :69]})
        K, V = c.update(k[:, :, 69:], v[:, :, 69:], 1, {"cos": zero["cos"][:, 69:], "sin": zero["sin"][:, 69:]})
        assert torch.equal(K, k) and torch.equal(V, v) and c.get_seq_length(1) == 70 and c.get_seq_length(0) == 0
        ex = KVCompCacheConfigStatic.extract_cache
        rnd = KVCompCachePytorchQuant.round_ - 1
        assert torch.equal(ex.key_caches[rnd][0], k) and torch.equal(ex.value_caches[rnd][0], v)
        c2 = KVCompCachePytorchQuant(B, H, D, 2)          # a later round with a prefill ends the collection
        with pytest.raises(JumpOutException):
            c2.update(k[:, :, :69], v[:, :, :69], 1, {"cos": zero["cos"][:, :69], "sin": zero["sin"][:, :69]})
    finally:
        KVCompCacheConfigStatic.extract_cache = None


def test_unset_config_raises():
    from kvcomp_amd.cache import KVCompCachePytorchQuant
    from kvcomp_amd.ctx import KVCompCacheConfigStatic
    KVCompCacheConfigStatic.config = None
    c = KVCompCachePytorchQuant(1, 1, 64, 1)
    with pytest.raises(ValueError):
        c.get_seq_length(0)
    with pytest.raises(ValueError):
        c.update(torch.zeros(1, 1, 1, 64), torch.zeros(1, 1, 1, 64), 0, {"cos": None, "sin": None})


def test_entropy_coded_backend_round_trips_within_the_error_bound():
    """KVCompCacheCuda: update() returns the decoded history; every element is within 0.53 * scale of the input
    (src/compute.cpp:60-69) and the tail is exact."""
    from kvcomp_amd.cache import KVCompCache
    from kvcomp_amd.compute import apply_rotary_pos_emb_single
    _set_config("BlockQuant", "TokenQuant", k_bs=64, v_bs=128, k_recent=64, v_recent=128)
    B, H, D, L = 1, 4, 128, 1
    steps = [300] + [1] * 70
    T = sum(steps)
    k = S.synth_k(T, B, H, D).permute(1, 2, 0, 3).contiguous()
    v = S.synth_v(T, B, H, D).permute(1, 2, 0, 3).contiguous()
    cos, sin = _rope(T, D)
    cache = KVCompCache(B, H, D, L, backend="encode")
    pos = 0
    for n_new in steps:
        kw = {"cos": cos[:, pos:pos + n_new].to(DEV), "sin": sin[:, pos:pos + n_new].to(DEV)}
        K, V = cache.update(k[:, :, pos:pos + n_new].to(DEV), v[:, :, pos:pos + n_new].to(DEV), 0, kw)
        pos += n_new
        assert cache.get_seq_length(0) == pos and K.shape == (B, H, pos, D) and V.shape == (B, H, pos, D)
    kr = torch.cat([apply_rotary_pos_emb_single(k[:, :, a:b], cos[:, a:b], sin[:, a:b]) for a, b in _chunks(steps)], dim=2)
    kctx, vctx = cache.cache_instance.k_cache_buffer[0], cache.cache_instance.v_cache_buffer[0]
    assert kctx.compressed_ctx_len == 320 and vctx.compressed_ctx_len == 256
    assert torch.equal(K[:, :, 320:].cpu(), kr[:, :, 320:]) and torch.equal(V[:, :, 256:].cpu(), v[:, :, 256:])
    k_range = (kr[:, :, :320].float().reshape(B, H, 5, 64, D).amax(dim=(1, 3, 4)) - kr[:, :, :320].float().reshape(B, H, 5, 64, D).amin(dim=(1, 3, 4)))
    assert (K[:, :, :320].cpu().float() - kr[:, :, :320].float()).abs().max() <= 0.53 * 0.1 * k_range.max() * 1.01
    assert (V[:, :, :256].cpu().float() - v[:, :, :256].float()).abs().max() <= 0.53 * 0.2 * (v.float().amax() - v.float().amin()) * 1.01
    assert math.isfinite(kctx.get_cr()) and kctx.get_cr() > 1.5
