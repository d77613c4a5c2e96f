"""Pins of the oracle's tile wire format (E1-E3, D1-D2, T3): a hand-worked tile, an independent model that
builds every lane stream as a Python bit string, the decoder's offset arithmetic
(kvcomp_cuda_extension/src/kernels.cu:598-600,620,635), and exact round trips."""
import numpy as np
import pytest

from oracle import oracle as O


def _table(book, n=None):
    """{symbol: '0101'} -> encode table bytes (include/huffman.h:13-16), index = symbol."""
    n = n or (max(book) + 1)
    t = np.zeros(n * 8, np.uint8)
    v = t.view(np.uint32)
    for s, c in book.items():
        v[2 * s], v[2 * s + 1] = int(c, 2), len(c)
    return t


def _tree(book):
    counts = np.zeros(256, np.int64)
    code = np.zeros(256, np.uint32)
    length = np.zeros(256, np.uint32)
    for s, c in book.items():
        counts[s], code[s], length[s] = 1, int(c, 2), len(c)
    st, tree = O.decode_tree(code, length, counts)
    assert st == 0
    return tree


BOOK3 = {0: "0", 1: "10", 2: "11"}


def test_hand_worked_k_tile():
    """Lane 0 = [1,0,2,0,...]: bits 10 0 11 + 125 zeros = 130 bits -> 17 bytes 98 00.., pad 6, info 17*8+6 = 142.
    Lane 1 = zeros: 128 bits -> 16 bytes, end 33, pad 0, info 264.  Every other lane: 16 bytes."""
    sym = np.zeros((1, 64, 1, 1, 128), np.uint8)
    sym[0, 0, 0, 0, :3] = [1, 0, 2]
    payload, bi, ti = O.encode_tiles(sym, True, _table(BOOK3), base_global_offset=1000)
    assert payload.size == 17 + 63 * 16
    assert payload[:17].tolist() == [0x98] + [0] * 16 and not payload[17:].any()
    info = ti.view(np.uint16)
    assert info[0] == 142 and info[1] == 264 and info[63] == (17 + 63 * 16) * 8
    assert bi.view(np.uint32)[0] == 1000 and bi.view(np.uint16)[2] == payload.size and bi.view(np.uint16)[3] == 0
    # decoder arithmetic: start = prev >> 3, bits = (end - start) * 8 - pad
    assert ((142 >> 3) - 0) * 8 - (142 & 7) == 130
    assert ((264 >> 3) - (142 >> 3)) * 8 - (264 & 7) == 128
    bi0 = bi.copy()
    bi0.view(np.uint32)[0] = 0
    assert np.array_equal(O.decode_tiles(payload, bi0, ti, _tree(BOOK3), sym.shape, True), sym)


def test_hand_worked_v_tile_geometry():
    """V: lane t <-> channel 64*col + t, symbol i <-> token i (kernels.cu:503-519).  One non-zero symbol at
    (token 5, channel 70) must land in tile 1, lane 6, symbol 5: stream = 5 zeros, '11', 122 zeros."""
    sym = np.zeros((1, 128, 1, 1, 128), np.uint8)
    sym[0, 5, 0, 0, 70] = 2
    payload, bi, ti = O.encode_tiles(sym, False, _table(BOOK3))
    assert bi.size == 2 * 8
    info = ti.view(np.uint16).reshape(2, 64)
    assert (np.diff(np.concatenate([[0], info[0] >> 3])) == 16).all()          # tile 0: all-zero lanes, 16 B each
    off1 = int(bi.view(np.uint32)[2])
    assert off1 == 64 * 16
    lane6 = payload[off1 + 6 * 16: off1 + 6 * 16 + 17]
    assert lane6.tolist() == [0b00000110] + [0] * 16                           # 00000 11 0...
    assert info[1, 6] == (6 * 16 + 17) * 8 + 7                                 # 129 bits -> 17 bytes, pad 7
    assert np.array_equal(O.decode_tiles(payload, bi, ti, _tree(BOOK3), sym.shape, False), sym)


def _string_model(sym5, is_k, book, vec_len):
    """Independent restatement: each lane stream is ''.join(codes) padded with '0' to a byte."""
    NB, BS, B, H, D = sym5.shape
    flat = sym5.reshape(NB * BS, B * H * D)
    tokens, stride = flat.shape
    rows = tokens // (64 if is_k else vec_len)
    cols = stride // (vec_len if is_k else 64)
    payload, infos, bnums = bytearray(), [], []
    for r in range(rows):
        for c in range(cols):
            end = 0
            for t in range(64):
                vec = flat[64 * r + t, vec_len * c: vec_len * (c + 1)] if is_k else flat[vec_len * r: vec_len * (r + 1), 64 * c + t]
                s = "".join(book[int(v)] for v in vec)
                pad = (-len(s)) % 8
                s += "0" * pad
                payload += int(s, 2).to_bytes(len(s) // 8, "big")
                end += len(s) // 8
                infos.append(end * 8 + pad)
            bnums.append(end)
    return bytes(payload), infos, bnums


@pytest.mark.parametrize("is_k,shape,vec_len", [(True, (2, 64, 1, 2, 128), 128), (False, (1, 128, 2, 1, 128), 128),
                                                (True, (1, 64, 2, 1, 96), 96), (False, (2, 128, 1, 2, 96), 128),
                                                (True, (1, 64, 1, 3, 64), 64)])
def test_encoder_equals_bit_string_model(is_k, shape, vec_len):
    rng = np.random.default_rng(9)
    sym = np.clip(np.rint(rng.standard_normal(shape) * 2.5 + 8), 0, 40).astype(np.uint8)
    book = O.py_huffman_codebook(sym)
    payload, bi, ti = O.encode_tiles(sym, is_k, _table(book, 41), 77, vec_len=vec_len)
    m_payload, m_infos, m_bnums = _string_model(sym, is_k, book, vec_len)
    assert payload.tobytes() == m_payload
    assert ti.view(np.uint16).tolist() == m_infos
    assert bi.view(np.uint16)[2::4].tolist() == m_bnums
    offs = bi.view(np.uint32)[0::2]
    assert offs.tolist() == (77 + np.concatenate([[0], np.cumsum(m_bnums)[:-1]])).tolist()
    bi0 = bi.copy()
    bi0.view(np.uint32)[0::2] -= 77
    assert np.array_equal(O.decode_tiles(payload, bi0, ti, _tree(book), shape, is_k, vec_len=vec_len), sym)


def test_decoder_rejects_truncated_stream():
    sym = np.ones((1, 64, 1, 1, 128), np.uint8)
    payload, bi, ti = O.encode_tiles(sym, True, _table(BOOK3))
    ti2 = ti.copy()
    ti2.view(np.uint16)[0] -= 8          # lane 0 loses a byte
    with pytest.raises(ValueError):
        O.decode_tiles(payload, bi, ti2, _tree(BOOK3), sym.shape, True)


def test_fused_reference_equals_numpy_on_dequantized_cache():
    from tests import _synth as S
    T, B, H, D, rep = 128, 2, 2, 64, 2
    x5 = S.np16(S.blocked(S.synth_k(T, B, H, D), 64))
    _, _, scale, sym, mn = O.quant(x5, O.MASK_CHANNEL, 0.1)
    q = S.np16(S.synth_q(B, H * rep, D))
    deq = O.dequant(sym, mn, scale, O.MASK_CHANNEL).reshape(T, B, H, D).astype(np.float64)
    ref = np.einsum("tbhd,bhd->bht", np.repeat(deq, rep, axis=2), q.astype(np.float64))
    assert np.allclose(O.fused_k(sym.reshape(T, B, H, D), mn, scale, O.MASK_CHANNEL, 64, q), ref, rtol=1e-12, atol=1e-12)
    x5 = S.np16(S.blocked(S.synth_v(T, B, H, D), 128))
    _, _, scale, sym, mn = O.quant(x5, O.MASK_V_TOKEN, 0.2)
    p = S.np16(S.synth_p(B, H * rep, T))
    deq = O.dequant(sym, mn, scale, O.MASK_V_TOKEN).reshape(T, B, H, D).astype(np.float64)
    ref = np.einsum("tbhd,bht->bhd", np.repeat(deq, rep, axis=2), p.astype(np.float64))
    assert np.allclose(O.fused_v(sym.reshape(T, B, H, D), mn, scale, O.MASK_V_TOKEN, 128, p), ref, rtol=1e-12, atol=1e-12)


def test_cpu_baseline_stream_walk_matches_exact_sum():
    from tests import _synth as S
    T, B, H, D = 128, 1, 2, 128
    x5 = S.np16(S.blocked(S.synth_k(T, B, H, D), 64))
    _, _, scale, sym, mn = O.quant(x5, O.MASK_K_BLOCK, 0.1)
    shift, enc, dec = O.build_codebook(sym)
    payload, bi, ti = O.encode_tiles(sym, True, enc)
    q = S.np16(S.synth_q(B, H, D))
    got = O.fused_k_from_stream(payload, bi, ti, dec, mn, scale, q, T, B * H * D)
    ref = O.fused_k(sym.reshape(T, B, H, D), mn, scale, O.MASK_K_BLOCK, 64, q).reshape(B * H, T)
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
