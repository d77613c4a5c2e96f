"""The one-pass tile encoder's look-back: no wave may wait for another before the sizes of all its own tiles are
published, whatever those sizes are; a wave that gives up on its look-back costs time, not the result.

The reference's encoder claims room for a tile with one atomic and cannot fail this way
(kvcomp_cuda_extension/src/kernels.cu:472-479); this build's keeps tile order and must be as safe."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S
from tests.test_gpu_ctx import _config, _oracle_mask

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _encode_direct(is_k, x, eb, table, one_pass, polls=None):
    """Fused quantize + encode of x [T, B, H, D] through kvc_encode_async; returns (payload, block_infos,
    thread_infos, result words) on the host."""
    from kvcomp_amd import _lib
    from kvcomp_amd import kvcomp_cuda as m
    T, B, H, D = x.shape
    mask = O.MASK_CHANNEL if is_k else O.MASK_V_TOKEN
    sizes = m.buffer_sizes(T, B * H * D, is_k, H, D)
    bi, ti = (torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes[:2])
    payload = torch.zeros(sizes[3], dtype=torch.uint8, device=DEV)
    groups = _lib.lib().kvc_quant_groups(T // 64, 64, B, H, D, mask)
    mn = torch.zeros(groups, dtype=torch.int8, device=DEV)
    sc = torch.zeros(groups, dtype=torch.float16, device=DEV)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    was = _lib.set_option("encode_one_pass", one_pass)
    was_polls = _lib.set_option("encode_lookback_polls", polls) if polls is not None else None
    try:
        m.encode_async(is_k, batch=B, head_num=H, head_dim=D, tokens=T, cache=x, quant_mask=mask, eb=eb, min_ints=mn, scales=sc,
                       encode_tables=table, table_bytes=table.numel(), block_infos=bi, thread_infos=ti, encoded=payload,
                       result=result)
        total = m.encode_result(result, payload.numel())[0]
    finally:
        _lib.set_option("encode_one_pass", was)
        if was_polls is not None:
            _lib.set_option("encode_lookback_polls", was_polls)
    return payload[:total].cpu().numpy(), bi.cpu().numpy(), ti.cpu().numpy(), result.cpu().numpy(), mn.cpu().numpy(), sc.cpu().numpy()


def _table_for(is_k, x, eb):
    """Encode table of the codebook of x's own symbols (every symbol the error bound allows counted once more)."""
    from kvcomp_amd.ctx import KVCompCtx
    T, B, H, D = x.shape
    ctx = KVCompCtx(is_k, B, H, D, eb)
    ctx.codebook_smoothing = True
    ctx.build_codebook([x[:min(T, 512)]])
    return ctx.encode_codebook.clone()


@pytest.mark.parametrize("is_k,eb,T,B,H,D", [
    (False, 0.2, 8192, 4, 16, 128),      # V, Gaussian, eb 0.2: tiles of about 2030 bytes, 8192 of them
    (True, 0.05, 4096, 4, 32, 128),      # K, head_dim 128, eb 0.05: tiles beyond 4096 bytes
    (True, 0.1, 8192, 2, 32, 96),        # the common case: tiles of about 2700 bytes
])
def test_look_back_never_waits_long_whatever_the_tile_size(is_k, eb, T, B, H, D):
    """Two tiles per wave over at least 8192 tiles whose payloads straddle 2048 / exceed 4096 bytes (the sizes up to
    which an earlier version of the kernel could hold a run's first tile back; a larger one it placed before the
    second was counted, so that each wave waited for the one before it: 18 ms for a 0.2 ms encode, some 21 000 looks
    per wave).  The most looks any wave needed stays small, and the bytes are those of the two-pass encoder."""
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D).to(DEV)
    table = _table_for(is_k, x, eb)
    pay1, bi1, ti1, res1, mn1, sc1 = _encode_direct(is_k, x, eb, table, one_pass=1)
    tiles = bi1.size // 8
    assert tiles >= 8192 and int(res1[4]) == tiles
    mean_tile = pay1.size / tiles
    assert (1900 < mean_tile < 2200) if not is_k else (mean_tile > 4096 if eb == 0.05 else mean_tile > 2048)
    print("tiles %d, mean payload %.0f B, most looks of one wave that found a word not ready: %d" % (tiles, mean_tile, res1[6]))
    assert 0 <= int(res1[6]) < 1500
    pay0, bi0, ti0, res0, mn0, sc0 = _encode_direct(is_k, x, eb, table, one_pass=0)
    assert int(res0[6]) == 0
    assert np.array_equal(pay1, pay0) and np.array_equal(bi1, bi0) and np.array_equal(ti1, ti0)
    assert np.array_equal(mn1, mn0) and np.array_equal(sc1.view(np.uint16), sc0.view(np.uint16))
    assert (int(res1[2]), int(res1[3])) == (int(res0[2]), int(res0[3]))


def _uniform(T, B, H, D, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.rand(T, B, H, D, generator=g) * 2.0 - 1.0).to(torch.float16)


@pytest.mark.parametrize("is_k,D", [(True, 128), (False, 128), (True, 96)])
@pytest.mark.parametrize("from_symbols", [False, True])
def test_two_payloads_that_do_not_fit_the_waves_lds_together(is_k, D, from_symbols):
    """Uniform data at an error bound of 1 / 120: some 120 symbols of about equal frequency, 7-bit codes, tiles of
    about 7 KB.  Two of those do not fit a wave's LDS area, so the kept tile is placed before the next one is packed
    (both sizes having been published first).  Payload and metadata must be the oracle's."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    T, B, H, eb = 1024, 1, 3, 1.0 / 120.0
    x = _uniform(T, B, H, D, 77).to(DEV)
    was = _lib.set_option("encode_one_pass", 3)                 # two tiles per wave, also from symbols
    try:
        ctx = KVCompCtx(is_k, B, H, D, eb)
        ctx.build_codebook([x])
        ctx.store(x, want_symbols=from_symbols)
        ctx.store(x, want_symbols=from_symbols)
    finally:
        _lib.set_option("encode_one_pass", was)
    o = O.quant(S.np16(S.blocked(x.cpu(), ctx.block_size)), _oracle_mask(ctx), eb)
    pay, bi, ti = O.encode_tiles(o[3], is_k, ctx.encode_codebook.cpu().numpy(), 0, vec_len=D if is_k else 128)
    sizes = bi.view(np.uint32).reshape(-1, 2)[:, 1]
    symbols_per_tile = 64 * D if is_k else 8192
    assert sizes.min() * 8 > 6.3 * symbols_per_tile and sizes.max() <= 8191     # no two of them fit 12.5 KB
    got_bi, got_ti, got = ctx.block_infos.cpu().numpy(), ctx.thread_infos.cpu().numpy(), ctx.encoded_data.cpu().numpy()
    assert np.array_equal(got_bi[:bi.size], bi) and np.array_equal(got_ti[:ti.size], ti)
    assert np.array_equal(got[:pay.size], pay) and np.array_equal(got[pay.size:2 * pay.size], pay)


@pytest.mark.parametrize("polls", [-1, 0])
@pytest.mark.parametrize("is_k,from_symbols,T,B,H,D", [(True, False, 1024, 2, 5, 128), (False, False, 1024, 2, 5, 96),
                                                       (True, True, 1024, 1, 7, 96), (False, True, 2048, 1, 4, 128)])
def test_a_look_back_that_gives_up_costs_time_not_the_result(is_k, from_symbols, T, B, H, D, polls):
    """encode_lookback_polls = 0: a wave gives up the first time it finds a word of its look-back not ready; -1: the
    call is treated as if one had.  Every kernel still ends normally, and the finishing kernel encodes the call again
    in two passes of its own: payload, metadata and totals are the oracle's, no error is reported, and a second store
    continues behind the first."""
    from kvcomp_amd import _lib
    from kvcomp_amd.ctx import KVCompCtx
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    eb = 0.1 if is_k else 0.2
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D, 9).to(DEV)
    was = _lib.set_option("encode_one_pass", 3), _lib.set_option("encode_lookback_polls", polls)
    try:
        ctx = KVCompCtx(is_k, B, H, D, eb)
        ctx.build_codebook([x])
        ctx.store(x, want_symbols=from_symbols)
        ctx.store(x, want_symbols=from_symbols)
    finally:
        _lib.set_option("encode_one_pass", was[0])
        _lib.set_option("encode_lookback_polls", was[1])
    o = O.quant(S.np16(S.blocked(x.cpu(), ctx.block_size)), _oracle_mask(ctx), eb)
    pay, bi, ti = O.encode_tiles(o[3], is_k, ctx.encode_codebook.cpu().numpy(), 0, vec_len=D if is_k else 128)
    got_bi, got_ti, got = ctx.block_infos.cpu().numpy(), ctx.thread_infos.cpu().numpy(), ctx.encoded_data.cpu().numpy()
    assert got.size == 2 * pay.size
    assert np.array_equal(got_bi[:bi.size], bi) and np.array_equal(got_ti[:ti.size], ti)
    assert np.array_equal(got[:pay.size], pay) and np.array_equal(got[pay.size:], pay)
    second = got_bi[bi.size:].view(np.uint32).reshape(-1, 2)
    first = bi.view(np.uint32).reshape(-1, 2)
    assert np.array_equal(second[:, 0], first[:, 0] + pay.size) and np.array_equal(second[:, 1], first[:, 1])
    assert ctx.max_tile_bytes == int(first[:, 1].max())
    assert np.array_equal(ctx.quant_scales.cpu().numpy().ravel().view(np.uint16)[:o[2].size], o[2].ravel().view(np.uint16))
    dec, _ = ctx.get_decode_quant_ints()
    assert np.array_equal(dec.cpu().numpy()[:o[3].shape[0]], o[3])


def test_forced_give_up_on_the_queued_path_leaves_no_error():
    """The same through kvc_encode_async (results stay on the device): error word clear, totals right."""
    _config(k_mode="ChannelQuant", v_mode="TokenQuant", k_recent=64, v_recent=128)
    x = S.synth_k(2048, 2, 4, 128, 3).to(DEV)
    table = _table_for(True, x, 0.1)
    want = _encode_direct(True, x, 0.1, table, one_pass=0)
    got = _encode_direct(True, x, 0.1, table, one_pass=3, polls=-1)
    for a, b in zip(want[:3], got[:3]):
        assert np.array_equal(a, b)
    assert int(got[3][1]) == 0 and int(got[3][0]) == want[0].size and tuple(got[3][2:5]) == tuple(want[3][2:5])
