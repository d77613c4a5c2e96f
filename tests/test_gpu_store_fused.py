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
]


def _data(is_k, T, B, H, D, dist, seed):
    if dist == "laplace":
        return S.synth_laplace(T, B, H, D, seed)
    return (S.synth_k if is_k else S.synth_v)(T, B, H, D, seed)


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
