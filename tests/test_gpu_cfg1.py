"""The codec round trip of the first benchmark configuration at its full size: one Llama-2-7B-shaped layer,
fp16 K and V of [32 heads, 1024 tokens, head_dim 128], K quantized per channel and V per token at eb = 0.1 over
64-token blocks, a Huffman codebook PER BLOCK, encode, decode, dequantize.

Checked per block: quantized symbols / minima / scales bit-exact against the oracle (itself pinned against stock
PyTorch fp16 ops); codebook and bitstream of the whole-tensor coder bit-exact against the stdlib-heapq model of
utils/huffman.py; the tile codec with that block's codebook restores the symbols exactly; the dequantized block is
bit-exact against the reference dequantizer's arithmetic; and the fused q.K^T over the 16 differently-coded blocks
(one decode table per tile row) matches fp32 attention scores to 1e-3."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
T, B, H, D, BS, EB = 1024, 1, 32, 128, 64, 0.1


def _ptr(t):
    return C.c_void_p(t.data_ptr())


@pytest.mark.parametrize("is_k", [True, False])
def test_per_block_codebooks_round_trip(is_k):
    import kvcomp_amd.kvcomp_cuda as m
    from kvcomp_amd import _lib
    from kvcomp_amd.compute import dequant, quant
    from kvcomp_amd.huffman import huffman_encode
    L = _lib.lib()
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D)
    mask = O.MASK_CHANNEL if is_k else O.MASK_V_TOKEN
    dims = [1] if is_k else [2, 3, 4]
    x5 = S.blocked(x, BS)                                            # [16, 64, 1, 32, 128]
    sym_d, min_d, scale_d = quant(x5.to(DEV), dims, EB)
    _, _, ref_scale, ref_sym, ref_min = O.quant(S.np16(x5), mask, EB)
    assert np.array_equal(sym_d.cpu().numpy(), ref_sym)
    assert np.array_equal(min_d.cpu().numpy().ravel(), ref_min.ravel())
    assert np.array_equal(scale_d.cpu().numpy().view(np.uint16).ravel(), ref_scale.view(np.uint16).ravel())
    # dequantized cache, bit for bit (RN16(f32(sym + min) * f32(scale)), utils/compute.py + kvcomp_encode.py:146)
    deq = dequant(sym_d, min_d, scale_d, dims)
    ref_deq = O.dequant(ref_sym, ref_min, ref_scale, mask)
    assert np.array_equal(deq.cpu().numpy().view(np.uint16), ref_deq.view(np.uint16))

    NB = T // BS
    rows_per_tile_row = 1 if is_k else 2                              # V tiles span 128 tokens = two blocks
    n_books = NB // rows_per_tile_row
    sizes = m.calculate_buffer_size(sym_d, is_k, H, D)
    bi = torch.zeros(sizes[0], dtype=torch.uint8, device=DEV)
    ti = torch.zeros(sizes[1], dtype=torch.uint8, device=DEV)
    payload = torch.zeros(sizes[3], dtype=torch.uint8, device=DEV)
    idx = torch.zeros(8, dtype=torch.uint8, device=DEV)
    trees, total_bits = [], 0
    bi_per, ti_per = sizes[0] // n_books, sizes[1] // n_books
    dec_fn = m.k_entropy_decode_cuda_export if is_k else m.v_entropy_decode_cuda_export
    for blk in range(NB):
        s_blk = sym_d[blk]
        # ---- the reference's whole-tensor coder on this block: codebook and bitstream
        bits, book = huffman_encode(s_blk)
        ref_book = O.py_huffman_codebook(ref_sym[blk])
        assert book == ref_book, "codebook of block %d" % blk
        assert np.array_equal(bits.cpu().numpy(), O.py_bits(ref_sym[blk], ref_book)), "bitstream of block %d" % blk
        total_bits += bits.numel()
    # ---- all codebooks and the whole encode in three launches on the stream, no host round trip in between:
    # per-codebook histograms -> Huffman codes and tables on the device -> one encode call that gives every tile
    # row its own table
    counts = m.symbol_counts_chunks(sym_d, n_books)
    enc_tabs, trees_d, meta = m.build_codebook_device(counts, m.TREE_I8)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    m.encode_async(is_k, batch=B, head_num=H, head_dim=D, tokens=T, symbols=sym_d, encode_tables=enc_tabs,
                   table_bytes=enc_tabs.shape[1], table_stride=enc_tabs.shape[1], rows_per_codebook=1, codebook_meta=meta,
                   block_infos=bi, thread_infos=ti, encoded=payload, result=result)
    used, max_tile, max_stream, tiles = m.encode_result(result, payload.numel())
    assert tiles == sizes[0] // 8 and 0 < max_stream <= max_tile <= 8191
    meta_h = meta.cpu().numpy()
    assert (meta_h[:, 3] == 0).all() and (meta_h[:, 0] == 0).all()
    # per codebook, against the oracle: the table, and this row's tiles encoded with it at the offset the rows
    # before it ended at
    pos = 0
    for book_i in range(n_books):
        rows = slice(book_i * rows_per_tile_row, (book_i + 1) * rows_per_tile_row)
        counts_h = np.bincount(ref_sym[rows].ravel(), minlength=256).astype(np.int64)
        code, length = O.huffman_build(counts_h)
        _, ref_tab = O.encode_table(code, length, counts_h)
        assert np.array_equal(enc_tabs[book_i, :int(meta_h[book_i, 1])].cpu().numpy(), ref_tab)
        assert not enc_tabs[book_i, int(meta_h[book_i, 1]):].any()
        # the host builder gives the same bytes (one construction serves both)
        shift, enc_tab, tree = m.build_codebook([sym_d[rows].contiguous()])
        assert shift == 0 and np.array_equal(enc_tab.numpy(), ref_tab)
        assert np.array_equal(trees_d[book_i, :int(meta_h[book_i, 2])].cpu().numpy(), tree.numpy())
        trees.append(tree)
        ref_payload, ref_bi, ref_ti = O.encode_tiles(ref_sym[rows], is_k, ref_tab, pos, vec_len=D if is_k else 128)
        assert np.array_equal(payload[pos:pos + ref_payload.size].cpu().numpy(), ref_payload), "payload of codebook %d" % book_i
        assert np.array_equal(bi[book_i * bi_per:(book_i + 1) * bi_per].cpu().numpy(), ref_bi)
        assert np.array_equal(ti[book_i * ti_per:(book_i + 1) * ti_per].cpu().numpy(), ref_ti)
        pos += ref_payload.size
        # ---- decode this row with its own tree, out of the shared payload buffer
        s_rows = sym_d[rows].contiguous()
        out = torch.zeros_like(s_rows)
        dec_fn(payload[:pos], bi[book_i * bi_per:(book_i + 1) * bi_per].clone(), ti[book_i * ti_per:(book_i + 1) * ti_per].clone(),
               tree.to(DEV), out, H, D)
        assert torch.equal(out, s_rows), "round trip of codebook %d" % book_i
    assert pos == used
    # entropy-coded size is within a byte per lane stream of the whole-tensor coder's bit count
    assert total_bits / 8 <= used <= total_bits / 8 + T * B * H * D / 128 + 64

    # ---- fused kernels over all rows at once, one decode table per tile row
    # (trees of different sizes: the tables are built one by one into one array)
    lut_bytes = int(L.kvc_lut_bytes())
    luts = torch.zeros(n_books * lut_bytes, dtype=torch.uint8, device=DEV)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for i, t in enumerate(trees):
        td = t.to(DEV)
        _lib.check(L.kvc_build_lut(_ptr(td), td.numel(), m.TREE_I8, 1, 0, C.c_void_p(luts.data_ptr() + i * lut_bytes), stream))
    enc_all = payload[:used]
    if is_k:
        q = S.synth_q(B, H, D).to(DEV)
        scores = torch.zeros(B, H, T, dtype=torch.float32, device=DEV)
        _lib.check(L.kvc_k_scores_lut(_ptr(luts), 1, _ptr(bi), bi.numel(), _ptr(ti), ti.numel(), _ptr(enc_all), enc_all.numel(),
                                      _ptr(min_d), _ptr(scale_d), mask, _ptr(q), _ptr(scores), 1, 0, 0, 0, T, B, H, H, D,
                                      None, stream))
        ref = torch.einsum("tbhd,bhd->bht", deq.reshape(T, B, H, D).float(), q.float())
        assert (scores - ref).abs().max() <= 1e-3 * ref.abs().max()
    else:
        p = S.synth_p(B, H, T).to(DEV)
        part = torch.zeros(T // 128, B, H, D, dtype=torch.float32, device=DEV)
        _lib.check(L.kvc_v_partials_lut(_ptr(luts), 1, _ptr(bi), bi.numel(), _ptr(ti), ti.numel(), _ptr(enc_all), enc_all.numel(),
                                        _ptr(min_d), _ptr(scale_d), mask, _ptr(p), _ptr(part), 1, 0, 0, 0, T, B, H, H, D,
                                        None, stream))
        ref = torch.einsum("tbhd,bht->bhd", deq.reshape(T, B, H, D).float(), p.float())
        assert (part.sum(0) - ref).abs().max() <= 1e-3 * ref.abs().max()
