"""Huffman codebooks built on the device (kvc_histogram_chunks + kvc_build_codebook_device) against the oracle's
construction (itself pinned against the reference's huffman.cpp and stdlib heapq) and against the host builder:
encode tables and decode trees byte for byte, for histograms that stress the heap's tie rule, plus the edge cases
the host builder rejects; then the per-block codebooks of the first benchmark configuration end to end (histograms,
codebooks and decode tables without a host round trip, one table per tile row in the fused kernel)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _histograms():
    rng = np.random.default_rng(77)
    hs = []
    for n in (2, 3, 5, 8, 16, 17, 31, 64):                        # all-equal counts: every merge is a tie
        h = np.zeros(256, np.int64); h[:n] = 7; hs.append(h)
    for n in (4, 11, 40, 64):                                     # small counts, many ties, gaps in the alphabet
        h = np.zeros(256, np.int64); idx = rng.choice(100, n, replace=False); h[idx] = rng.integers(1, 4, n); hs.append(h)
    for sigma in (1.0, 2.5, 6.0, 15.0):                           # Gaussian-shaped (what quantized caches look like)
        x = np.clip(np.rint(rng.normal(30, sigma, 200000)), 0, 127).astype(np.int64); hs.append(np.bincount(x, minlength=256))
    h = np.zeros(256, np.int64); h[3] = 1; h[90] = 10 ** 12; hs.append(h)          # two symbols, far apart
    h = np.zeros(256, np.int64); h[:20] = [1, 1, 2, 3, 5, 8, 13, 21, 34, 55, 89, 144, 233, 377, 610, 987, 1597, 2584, 4181, 6765]
    hs.append(h)                                                                    # Fibonacci: a 19-bit code
    return hs


@pytest.mark.parametrize("fmt_name", ["TREE_I8", "TREE_I16"])
def test_device_codebooks_equal_oracle_and_host_builder(fmt_name):
    import kvcomp_amd.kvcomp_cuda as m
    fmt = getattr(m, fmt_name)
    hs = _histograms()
    enc, trees, meta = m.build_codebook_device(torch.from_numpy(np.stack(hs)).to(DEV), fmt)
    enc, trees, meta = enc.cpu().numpy(), trees.cpu().numpy(), meta.cpu().numpy()
    for i, h in enumerate(hs):
        code, length = O.huffman_build(h)
        shift, ref_tab = O.encode_table(code, length, h)
        st, ref_tree = O.decode_tree(code, length, h)
        if st != 0:                                      # more nodes than the int8 tree holds: wide format only
            if fmt == m.TREE_I8:
                assert meta[i, 3] == 4 and not enc[i].any()
                continue
            h_shift, h_tab, h_tree = m.build_codebook_from_counts(torch.from_numpy(h), fmt)
            assert tuple(meta[i]) == (h_shift, h_tab.numel(), h_tree.numel(), 0), i
            assert np.array_equal(enc[i, :ref_tab.size], ref_tab) and np.array_equal(trees[i, :h_tree.numel()], h_tree.numpy())
            continue
        if fmt == m.TREE_I16:                            # the same nodes, children as int16 (5-byte nodes)
            n8 = ref_tree.reshape(-1, 3)
            wide = np.zeros((n8.shape[0], 5), np.uint8)
            wide[:, 0] = n8[:, 0]
            wide[:, 1:3] = n8[:, 1].view(np.int8).astype("<i2").reshape(-1, 1).view(np.uint8)
            wide[:, 3:5] = n8[:, 2].view(np.int8).astype("<i2").reshape(-1, 1).view(np.uint8)
            ref_tree = wide.ravel()
        assert tuple(meta[i]) == (shift, ref_tab.size, ref_tree.size, 0), i
        assert np.array_equal(enc[i, :ref_tab.size], ref_tab), i
        assert not enc[i, ref_tab.size:].any()
        assert np.array_equal(trees[i, :ref_tree.size], ref_tree), i
        h_shift, h_tab, h_tree = m.build_codebook_from_counts(torch.from_numpy(h), fmt)
        assert h_shift == shift and np.array_equal(h_tab.numpy(), ref_tab) and np.array_equal(h_tree.numpy(), ref_tree)


def test_device_codebook_status_codes():
    import kvcomp_amd.kvcomp_cuda as m
    lone = np.zeros(256, np.int64); lone[5] = 9
    empty = np.zeros(256, np.int64)
    wide = np.zeros(256, np.int64); wide[:200] = np.arange(1, 201)                 # 200 symbols: too many nodes for int8
    high = np.zeros(256, np.int64); high[[3, 200]] = 1                             # a symbol above 127
    fib = np.zeros(256, np.int64)
    a, b = 1, 1
    for s in range(40):                                                            # 40 Fibonacci counts: a 39-bit code
        fib[s] = a; a, b = b, a + b
    cases = np.stack([lone, empty, wide, high, fib])
    _, _, meta8 = m.build_codebook_device(torch.from_numpy(cases).to(DEV), m.TREE_I8)
    enc16, _, meta16 = m.build_codebook_device(torch.from_numpy(cases).to(DEV), m.TREE_I16)
    assert meta8.cpu().numpy()[:, 3].tolist() == [1, 1, 4, 4, 2]
    assert meta16.cpu().numpy()[:, 3].tolist() == [1, 1, 0, 0, 2]
    assert not enc16.cpu().numpy()[[0, 1, 4]].any()
    for h in (lone, wide, fib):                                                    # the host builder refuses the same inputs
        with pytest.raises(RuntimeError):
            m.build_codebook_from_counts(torch.from_numpy(h), m.TREE_I8)


def test_chunked_histograms():
    import kvcomp_amd.kvcomp_cuda as m
    rng = np.random.default_rng(3)
    for n_chunks, chunk in ((1, 1000), (16, 64 * 4096), (5, 12345), (3, 7)):
        sym = rng.integers(0, 256, size=n_chunks * chunk, dtype=np.uint8)
        sym[: chunk // 2] = 17                                                     # a heavily skewed chunk
        got = m.symbol_counts_chunks(torch.from_numpy(sym).to(DEV), n_chunks).cpu().numpy()
        ref = np.stack([np.bincount(sym[c * chunk:(c + 1) * chunk], minlength=256) for c in range(n_chunks)])
        assert np.array_equal(got, ref)


def test_per_block_codebooks_without_a_host_round_trip():
    """K of the first benchmark configuration (32 heads x 128, 1024 tokens, one codebook per 64-token block):
    histograms, codebooks and decode tables are produced by three launches on the stream, each block is encoded with
    its own table, and the fused q.K^T with one decode table per tile row matches fp32 scores over the dequantized
    cache to 1e-3."""
    import kvcomp_amd.kvcomp_cuda as m
    from kvcomp_amd import _lib
    from kvcomp_amd.compute import dequant, quant
    L = _lib.lib()
    T, B, H, D, EB = 1024, 1, 32, 128, 0.1
    x5 = S.blocked(S.synth_k(T, B, H, D), 64)
    sym, mn, scale = quant(x5.to(DEV), [1], EB)
    NB = T // 64
    counts = m.symbol_counts_chunks(sym, NB)
    enc, trees, meta = m.build_codebook_device(counts, m.TREE_I8)
    lut_bytes = int(L.kvc_lut_bytes())
    luts = torch.zeros(NB * lut_bytes, dtype=torch.uint8, device=DEV)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(L.kvc_build_lut(C.c_void_p(trees.data_ptr()), trees.shape[1], m.TREE_I8, NB, trees.shape[1],
                               C.c_void_p(luts.data_ptr()), stream))
    meta_h = meta.cpu().numpy()                                                    # (only the test looks at the sizes)
    assert (meta_h[:, 3] == 0).all() and (meta_h[:, 0] == 0).all()
    ref_sym = sym.cpu().numpy()
    for blk in range(NB):
        h = np.bincount(ref_sym[blk].ravel(), minlength=256).astype(np.int64)
        code, length = O.huffman_build(h)
        _, ref_tab = O.encode_table(code, length, h)
        assert np.array_equal(enc[blk, :ref_tab.size].cpu().numpy(), ref_tab)
    sizes = m.calculate_buffer_size(sym, True, H, D)
    bi = torch.zeros(sizes[0], dtype=torch.uint8, device=DEV)
    ti = torch.zeros(sizes[1], dtype=torch.uint8, device=DEV)
    payload = torch.zeros(sizes[3], dtype=torch.uint8, device=DEV)
    # one call encodes all sixteen blocks, each tile row with the table of its own codebook, straight from the
    # tables the device builder wrote (a codebook that was not built would flag the call on the device)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    m.encode_async(True, batch=B, head_num=H, head_dim=D, tokens=T, symbols=sym, encode_tables=enc, table_bytes=enc.shape[1],
                   table_stride=enc.shape[1], rows_per_codebook=1, codebook_meta=meta, block_infos=bi, thread_infos=ti,
                   encoded=payload, result=result)
    used = m.encode_result(result, payload.numel())[0]
    pos = 0
    for blk in range(NB):                                                          # per block, against the oracle's encoder
        h = np.bincount(ref_sym[blk].ravel(), minlength=256).astype(np.int64)
        code, length = O.huffman_build(h)
        _, ref_tab = O.encode_table(code, length, h)
        ref_payload, ref_bi, ref_ti = O.encode_tiles(ref_sym[blk:blk + 1], True, ref_tab, pos, vec_len=D)
        assert np.array_equal(payload[pos:pos + ref_payload.size].cpu().numpy(), ref_payload)
        pos += ref_payload.size
    assert pos == used
    q = S.synth_q(B, H, D).to(DEV)
    scores = torch.zeros(B, H, T, dtype=torch.float32, device=DEV)
    enc_all = payload[:used]
    p = lambda t: C.c_void_p(t.data_ptr())
    _lib.check(L.kvc_k_scores_lut(p(luts), 1, p(bi), bi.numel(), p(ti), ti.numel(), p(enc_all), enc_all.numel(), p(mn), p(scale),
                                  O.MASK_CHANNEL, p(q), p(scores), 1, 0, 0, 0, T, B, H, H, D, None, stream))
    deq = dequant(sym, mn, scale, [1])
    ref = torch.einsum("tbhd,bhd->bht", deq.reshape(T, B, H, D).float(), q.float())
    assert (scores - ref).abs().max() <= 1e-3 * ref.abs().max()
