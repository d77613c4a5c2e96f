"""KVCompHFCache under a stock `transformers` Llama: the Cache contract (sequence lengths, shapes, growth one
token at a time), the dense (K, V) that update() hands back against a CPU replay of quantize -> dequantize made
of PyTorch's own fp16 ops, attention on the compressed streams against dense attention, and generation."""
import math

import pytest
import torch

from tests import _synth as S
from tests.test_gpu_cache import _expected

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _config(ebk=0.1, ebv=0.2):
    from kvcomp_amd.compute import QuantMode
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic
    KVCompCacheConfigStatic.config = KVCompCacheConfig("hf", QuantMode.ChannelQuant, QuantMode.TokenQuant, 64, 128, 64, 128,
                                                       ebk, ebv)


def test_layer_update_returns_the_quantized_history_bit_exact():
    from kvcomp_amd.hf_adapter import KVCompHFCache
    _config()
    B, H, D, L = 1, 4, 64, 2
    steps = [150] + [1] * 140
    T = sum(steps)
    ks = [S.synth_k(T, B, H, D, seed=31 + l).permute(1, 2, 0, 3).contiguous() for l in range(L)]
    vs = [S.synth_v(T, B, H, D, seed=41 + l).permute(1, 2, 0, 3).contiguous() for l in range(L)]
    cache = KVCompHFCache(L)
    assert cache.get_seq_length() == 0
    pos = 0
    for n_new in steps:
        for l in range(L):
            K, V = cache.update(ks[l][:, :, pos:pos + n_new].to(DEV), vs[l][:, :, pos:pos + n_new].to(DEV), l)
        pos += n_new
        assert cache.get_seq_length(L - 1) == pos and K.shape == (B, H, pos, D) and V.shape == (B, H, pos, D)
        assert cache.get_mask_sizes(1, 0) == (pos + 1, 0)
    for l in range(L):
        K, V = cache.layers[l].keys, cache.layers[l].values
        # K: per channel over 64-token blocks; V: per token over heads x channels (batch 1: the kernel path's groups)
        ek, kd = _expected(ks[l], 64, 64, 0.1, "ChannelQuant", steps)
        ev, vd = _expected(vs[l], 128, 128, 0.2, "TokenQuant", steps)
        assert kd == cache.layers[l].k_ctx.compressed_ctx_len and vd == cache.layers[l].v_ctx.compressed_ctx_len
        assert torch.equal(K.cpu().view(torch.int16), ek.view(torch.int16))
        assert torch.equal(V.cpu().view(torch.int16), ev.view(torch.int16))
    assert cache.compression_ratio() > 1.5


def _tiny_llama():
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=256, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=1024, attn_implementation="eager")
    return LlamaForCausalLM(cfg).to(DEV).to(torch.float16).eval()


@pytest.mark.parametrize("ebk,ebv,floor", [(0.1, 0.2, 0.9), (0.02, 0.02, 0.995)])
def test_decode_steps_track_the_dense_cache_within_the_error_bound(ebk, ebv, floor):
    """Logits of a random-init model (flat, hence sensitive) with the compressed cache against the dense cache:
    close at the benchmark error bounds, and converging as the bounds shrink."""
    from transformers import DynamicCache
    from kvcomp_amd.hf_adapter import KVCompHFCache
    _config(ebk, ebv)
    model = _tiny_llama()
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(0, 256, (1, 330), generator=g).to(DEV)
    ours, dense = KVCompHFCache(), DynamicCache()
    sims = []
    with torch.no_grad():
        model(ids[:, :256], past_key_values=ours, use_cache=True)
        model(ids[:, :256], past_key_values=dense, use_cache=True)
        for t in range(256, 330):
            a = model(ids[:, t:t + 1], past_key_values=ours, use_cache=True).logits[0, -1].float()
            b = model(ids[:, t:t + 1], past_key_values=dense, use_cache=True).logits[0, -1].float()
            sims.append(float(torch.nn.functional.cosine_similarity(a, b, dim=0)))
    assert ours.get_seq_length() == dense.get_seq_length() == 330
    assert ours.layers[0].k_ctx.compressed_ctx_len >= 256 and ours.layers[0].v_ctx.compressed_ctx_len >= 128
    assert min(sims) > floor, min(sims)
    # attention computed on the compressed streams equals dense attention over what update() returns
    layer = ours.layers[1]
    q = S.synth_q(1, 4, 64).to(DEV)
    out = layer.attend(q)
    K = layer.keys.float().repeat_interleave(2, dim=1)
    V = layer.values.float().repeat_interleave(2, dim=1)
    s = torch.einsum("bhd,bhtd->bht", q.float(), K) / math.sqrt(64)
    ref = torch.einsum("bht,bhtd->bhd", torch.softmax(s, dim=-1), V)
    assert float((out - ref).abs().max()) <= 1e-3 * float(ref.abs().max())


def test_generate_with_the_compressed_cache():
    from kvcomp_amd.hf_adapter import KVCompHFCache
    _config()
    model = _tiny_llama()
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 256, (1, 200), generator=g).to(DEV)
    cache = KVCompHFCache()
    out = model.generate(ids, past_key_values=cache, max_new_tokens=80, do_sample=False, use_cache=True, pad_token_id=0)
    assert out.shape == (1, 280) and cache.get_seq_length() == 279
    assert cache.layers[0].k_ctx.compressed_ctx_len == 256 and cache.layers[0].v_ctx.compressed_ctx_len == 256   # (279 - 279 % bs) / bs + 1 - recent / bs blocks


def test_model_attends_on_the_compressed_cache_through_the_attention_registry():
    """With the attention implementation "kvcomp" and a cache built with attend_compressed=True, single-token steps
    never decompress the history: update() stores the token and the registered attention function runs the fused
    decode attention of the layer.  Logits must agree with the same model reading the dense (K, V) that the
    compressed cache hands out otherwise (the two differ only by fp16 rounding of the dequantized cache and of
    the stock attention's arithmetic); prompts still take the dense path."""
    from kvcomp_amd import hf_adapter as HA
    _config(0.1, 0.2)
    model = _tiny_llama()
    name = HA.register_kvcomp_attention()
    g = torch.Generator().manual_seed(9)
    B = 2
    ids = torch.randint(0, 256, (B, 300), generator=g).to(DEV)
    dense_like, lazy = HA.KVCompHFCache(), HA.KVCompHFCache(attend_compressed=True)
    calls = {"n": 0}
    real_attend = HA.KVCompLayer.attend

    def counting_attend(self, *a, **k):
        calls["n"] += 1
        return real_attend(self, *a, **k)

    HA.KVCompLayer.attend = counting_attend
    try:
        sims, diffs = [], []
        with torch.no_grad():
            model.set_attn_implementation("sdpa")
            model(ids[:, :256], past_key_values=dense_like, use_cache=True)
            model.set_attn_implementation(name)
            model(ids[:, :256], past_key_values=lazy, use_cache=True)          # a prompt: dense path, no attend() call
            assert calls["n"] == 0
            for t in range(256, 300):
                model.set_attn_implementation("sdpa")
                a = model(ids[:, t:t + 1], past_key_values=dense_like, use_cache=True).logits[:, -1].float()
                model.set_attn_implementation(name)
                b = model(ids[:, t:t + 1], past_key_values=lazy, use_cache=True).logits[:, -1].float()
                sims.append(float(torch.nn.functional.cosine_similarity(a, b, dim=-1).min()))
                diffs.append(float((a - b).abs().max() / a.abs().max()))
        n_layers = model.config.num_hidden_layers
        assert calls["n"] == 44 * n_layers                                      # every decode step of every layer
        assert lazy.get_seq_length() == dense_like.get_seq_length() == 300
        assert all(layer.keys is None for layer in lazy.layers)                  # no dense history was produced
        assert min(sims) > 0.999 and max(diffs) < 2e-2, (min(sims), max(diffs))
        # and generation runs end to end
        model.set_attn_implementation(name)
        cache = HA.KVCompHFCache(attend_compressed=True)
        out = model.generate(ids[:, :200], past_key_values=cache, max_new_tokens=40, do_sample=False, use_cache=True)
        assert out.shape == (B, 240) and cache.get_seq_length() == 239
    finally:
        HA.KVCompLayer.attend = real_attend


def _tiny(family):
    import transformers as tf
    torch.manual_seed(0)
    if family == "mistral":                                   # grouped-query attention, 4 query heads per KV head
        cfg = tf.MistralConfig(vocab_size=256, hidden_size=512, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
                               num_key_value_heads=2, head_dim=64, max_position_embeddings=1024, sliding_window=None,
                               attn_implementation="sdpa")
        return tf.MistralForCausalLM(cfg).to(DEV).to(torch.float16).eval()
    if family == "phi3":                                      # head_dim 96, fused qkv projection
        cfg = tf.Phi3Config(vocab_size=256, hidden_size=384, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                            num_key_value_heads=4, max_position_embeddings=1024, original_max_position_embeddings=1024,
                            sliding_window=None, pad_token_id=0, attn_implementation="sdpa")
        return tf.Phi3ForCausalLM(cfg).to(DEV).to(torch.float16).eval()
    raise ValueError(family)


@pytest.mark.parametrize("family", ["mistral", "phi3"])
def test_other_architectures_attend_on_the_compressed_cache(family):
    """The model families the reference forks (models/mistral.py, models/phi3.py), as stock transformers code: grouped
    queries (4 per KV head) and head_dim 96 go through the same registered attention function."""
    from kvcomp_amd import hf_adapter as HA
    _config(0.1, 0.2)
    model = _tiny(family)
    name = HA.register_kvcomp_attention()
    g = torch.Generator().manual_seed(19)
    ids = torch.randint(1, 256, (2, 290), generator=g).to(DEV)
    dense_like, lazy = HA.KVCompHFCache(), HA.KVCompHFCache(attend_compressed=True)
    sims = []
    with torch.no_grad():
        model.set_attn_implementation("sdpa")
        model(ids[:, :256], past_key_values=dense_like, use_cache=True)
        model.set_attn_implementation(name)
        model(ids[:, :256], past_key_values=lazy, use_cache=True)
        for t in range(256, 290):
            model.set_attn_implementation("sdpa")
            a = model(ids[:, t:t + 1], past_key_values=dense_like, use_cache=True).logits[:, -1].float()
            model.set_attn_implementation(name)
            b = model(ids[:, t:t + 1], past_key_values=lazy, use_cache=True).logits[:, -1].float()
            sims.append(float(torch.nn.functional.cosine_similarity(a, b, dim=-1).min()))
    assert all(layer.keys is None for layer in lazy.layers) and lazy.get_seq_length() == 290
    assert min(sims) > 0.999, min(sims)
