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
