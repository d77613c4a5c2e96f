"""The compiled `kvcomp_cuda` extension module (kvcomp_amd/ext/kvcomp_cuda.so, a PyTorch C++ extension over the C ABI):
the reference's module name, four constants and nine functions (kvcomp_cuda_extension/export_kvcomp.cpp:8-26,
kvcomp_cuda.pyi:14-84).  CPU tests: it loads, exports every name and refuses bad arguments with an exception.
GPU test: the reference's own call sequence (models/cache/kvcomp_encode.py:86-166: codebook -> buffer sizes ->
encode -> decode -> fused products) through the compiled module, bit-exact against the CPU oracle for the byte
results and within 1e-3 of max|reference| for the fused products (the reference's own check uses 1e-2,
evaluation/cr_throughput_eval.py:18-20)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S

NAMES = ("build_codebook", "calculate_buffer_size", "k_entropy_encode_cuda_export", "v_entropy_encode_cuda_export",
         "k_entropy_decode_cuda_export", "v_entropy_decode_cuda_export", "k_decode_and_mat_vec_mul_cuda_export",
         "v_decode_and_mat_vec_mul_cuda_export", "k_mat_vec_mul_cuda_export")
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ext():
    from kvcomp_amd import build
    if not os.path.exists(build.MODULE_PATH):          # normally built beforehand (python -m kvcomp_amd.build)
        assert os.path.exists(build.LIBPATH), "libkvcomp_hip.so is not built: run python -m kvcomp_amd.build"
        build.build_module(verbose=False)
    spec = importlib.util.spec_from_file_location("kvcomp_cuda", build.MODULE_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_module_exports_the_reference_names(ext):
    assert ext.__name__ == "kvcomp_cuda"
    assert (ext.K_VEC_LEN, ext.K_VEC_PER_BLK, ext.V_VEC_LEN, ext.V_VEC_PER_BLK) == (128, 64, 128, 64)
    for name in NAMES:
        assert callable(getattr(ext, name)), name


def test_buffer_sizes_agree_with_the_reference_formula(ext):
    """src/kernels.cu:893-917; needs no device."""
    import kvcomp_amd.kvcomp_cuda as m
    for shape, is_k, H, D in (((16, 64, 1, 32, 128), True, 32, 128), ((8, 128, 1, 32, 128), False, 32, 128),
                              ((2, 128, 2, 2, 64), False, 2, 64), ((4, 64, 2, 3, 96), True, 3, 96)):
        x = torch.empty(shape, dtype=torch.uint8)
        got = ext.calculate_buffer_size(x, is_k, H, D)
        assert got == m.calculate_buffer_size(x, is_k, H, D)
        tokens, stride = shape[0] * shape[1], shape[2] * shape[3] * shape[4]
        tiles = tokens * stride // (64 * D if is_k else 128 * 64)
        assert got == (tiles * 8, tiles * 64 * 2, 8, tokens * stride)


def test_bad_arguments_raise_instead_of_aborting(ext):
    """The reference aborts the process on a failed check (include/utils.h:7-15); here the caller gets an exception."""
    u8 = torch.zeros(64, dtype=torch.uint8)
    sym = torch.zeros(1, 64, 1, 1, 128, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="device tensor"):
        ext.k_entropy_encode_cuda_export(sym, u8, u8, u8, u8, u8, 0, 1, 128)
    with pytest.raises(RuntimeError, match="device tensor"):
        ext.v_entropy_decode_cuda_export(u8, u8, u8, u8, sym, 1, 128)
    with pytest.raises(RuntimeError, match="NB, BS, B, H, D"):
        ext.calculate_buffer_size(u8, True, 1, 128)
    with pytest.raises(RuntimeError, match="must not be empty"):
        ext.build_codebook([])
    h = torch.zeros(64, 1, 1, 128, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="Head num"):
        ext.k_mat_vec_mul_cuda_export(h, torch.zeros(1, 2, 128, dtype=torch.float16), torch.zeros(64, 1, 1, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="device tensor"):
        ext.k_mat_vec_mul_cuda_export(h, torch.zeros(1, 1, 128, dtype=torch.float16), torch.zeros(64, 1, 1, dtype=torch.float16))


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.to(DEV)


@pytest.mark.gpu
@pytest.mark.parametrize("is_k", [True, False])
@pytest.mark.parametrize("shape", [(512, 1, 4, 128), (256, 2, 3, 64)])
def test_the_reference_call_sequence_through_the_compiled_module(ext, is_k, shape):
    T, B, H, D = shape
    bs, eb = (64, 0.1) if is_k else (128, 0.2)
    mask = O.MASK_K_BLOCK if is_k else O.MASK_V_TOKEN
    x = (S.synth_k if is_k else S.synth_v)(T, B, H, D)
    _, _, scale, sym, mn = O.quant(S.np16(S.blocked(x, bs)), mask, eb)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts)
    _, ref_enc = O.encode_table(code, length, counts)
    _, ref_dec = O.decode_tree(code, length, counts)
    sym_d = _dev(sym)

    shift, enc_tab, tree = ext.build_codebook([sym_d[: sym.shape[0] // 2], sym_d[sym.shape[0] // 2:]])
    assert shift == 0 and not enc_tab.is_cuda and not tree.is_cuda
    assert np.array_equal(enc_tab.numpy(), ref_enc) and np.array_equal(tree.numpy(), ref_dec)

    sizes = ext.calculate_buffer_size(sym_d, is_k, H, D)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    enc_fn = ext.k_entropy_encode_cuda_export if is_k else ext.v_entropy_encode_cuda_export
    base = 777
    payload, bi, ti = enc_fn(sym_d, enc_tab.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], base, H, D)
    ref_payload, ref_bi, ref_ti = O.encode_tiles(sym, is_k, ref_enc, base, vec_len=D if is_k else 128)
    assert payload.data_ptr() == bufs[3].data_ptr() and payload.numel() == ref_payload.size
    assert np.array_equal(payload.cpu().numpy(), ref_payload)
    assert np.array_equal(bi.cpu().numpy(), ref_bi) and np.array_equal(ti.cpu().numpy(), ref_ti)

    # decode reads payload offsets relative to the start of the buffer the encoder was given `base` for
    payload0, bi0, ti0 = enc_fn(sym_d, enc_tab.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
    out = torch.full(sym.shape, 0xAB, dtype=torch.uint8, device=DEV)
    dec_fn = ext.k_entropy_decode_cuda_export if is_k else ext.v_entropy_decode_cuda_export
    ms = dec_fn(payload0, bi0, ti0, tree.to(DEV), out, H, D)
    assert isinstance(ms, float) and ms >= 0.0
    assert torch.equal(out, sym_d)

    mn_d, scale_d = _dev(mn.ravel()), _dev(scale.ravel().view(np.uint16), torch.float16)
    if is_k:
        q = S.synth_q(B, H, D)
        scores = torch.zeros(B, H, T, dtype=torch.float16, device=DEV)
        ms = ext.k_decode_and_mat_vec_mul_cuda_export(tree.to(DEV), bi0, ti0, payload0, mn_d, scale_d, q.to(DEV), scores, H, D)
        ref = O.fused_k(sym.reshape(T, B, H, D), mn, scale, mask, bs, S.np16(q))
        assert ms >= 0.0 and np.abs(scores.float().cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()
        # dense baseline over the dequantized cache
        deq = torch.from_numpy(O.dequant(sym, mn, scale, mask)).reshape(T, B, H, D)
        dense = torch.zeros(T, B, H, dtype=torch.float16, device=DEV)
        ext.k_mat_vec_mul_cuda_export(deq.to(DEV), q.to(DEV), dense)
        want = torch.einsum("tbhd,bhd->tbh", deq.float(), q.float())
        assert (dense.float().cpu() - want).abs().max() <= 1e-3 * want.abs().max()
    else:
        p = torch.softmax(torch.randn(B, H, T, generator=torch.Generator().manual_seed(3)), dim=-1).to(torch.float16)
        part = torch.zeros(T // 128, B, H, D, dtype=torch.float16, device=DEV)
        ms = ext.v_decode_and_mat_vec_mul_cuda_export(tree.to(DEV), bi0, ti0, payload0, mn_d, scale_d, p.to(DEV), part, H, D)
        ref = O.fused_v(sym.reshape(T, B, H, D), mn, scale, mask, bs, p.numpy())
        got = part.float().sum(dim=0).cpu().numpy()
        assert ms >= 0.0 and np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()


@pytest.mark.gpu
def test_compiled_module_runs_on_the_current_stream(ext):
    """Work queued on a side stream before the call must be seen by it (the reference uses the legacy default stream)."""
    T, B, H, D = 256, 1, 2, 128
    x = S.synth_k(T, B, H, D)
    _, _, scale, sym, mn = O.quant(S.np16(S.blocked(x, 64)), O.MASK_K_BLOCK, 0.1)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sym_d = _dev(sym)
        shift, enc_tab, tree = ext.build_codebook([sym_d])
        sizes = ext.calculate_buffer_size(sym_d, True, H, D)
        bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
        payload, bi, ti = ext.k_entropy_encode_cuda_export(sym_d, enc_tab.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
        out = torch.zeros_like(sym_d)
        ext.k_entropy_decode_cuda_export(payload, bi, ti, tree.to(DEV), out, H, D)
    side.synchronize()
    assert torch.equal(out.cpu(), torch.from_numpy(sym))
