"""GPU parity tests: every HIP entry point (through kvcomp_amd.kvcomp_cuda -> C ABI) against the CPU oracle
on the same seeded inputs.  Integer/byte results must be bit-exact; fused attention pieces must be within
1e-3 of max|reference| (the reference's own check uses 1e-2, evaluation/cr_throughput_eval.py:18-20)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import _synth as S

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def kc():
    import kvcomp_amd.kvcomp_cuda as m
    return m


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.to(DEV)


def _make_stream(x_tbhd, is_k, eb, mask, block_size, tree_format=3):
    """Oracle pipeline: quantize -> codebook -> tile encode.  Returns a dict of numpy arrays."""
    x5 = S.np16(S.blocked(x_tbhd, block_size))
    _, _, scale, sym, mn = O.quant(x5, mask, eb)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts)
    shift, enc = O.encode_table(code, length, counts)
    assert shift == 0
    st, dec = O.decode_tree(code, length, counts)
    assert st == 0
    D = x_tbhd.shape[3]
    payload, bi, ti = O.encode_tiles(sym, is_k, enc, 0, vec_len=D if is_k else 128)
    return dict(x5=x5, sym=sym, mn=mn, scale=scale, enc=enc, dec=dec, payload=payload, bi=bi, ti=ti,
                code=code, length=length, counts=counts)


SHAPES = [(256, 1, 4, 128), (128, 2, 2, 128), (256, 1, 3, 64), (256, 2, 2, 96), (128, 1, 8, 72), (256, 2, 4, 40)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("is_k", [True, False])
def test_entropy_decode_matches_oracle(shape, is_k):
    T, B, H, D = shape
    x = S.synth_k(T, B, H, D) if is_k else S.synth_v(T, B, H, D)
    bs = 64 if is_k else 128
    s = _make_stream(x, is_k, 0.1, O.MASK_K_BLOCK if is_k else O.MASK_V_TOKEN, bs)
    # the oracle's own decoder must round-trip first
    assert np.array_equal(O.decode_tiles(s["payload"], s["bi"], s["ti"], s["dec"], s["sym"].shape, is_k, vec_len=D if is_k else 128), s["sym"])
    m = kc()
    out = torch.full(s["sym"].shape, 0xAB, dtype=torch.uint8, device=DEV)
    fn = m.k_entropy_decode_cuda_export if is_k else m.v_entropy_decode_cuda_export
    ms = fn(_dev(s["payload"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["dec"]), out, H, D)
    assert ms >= 0.0
    assert np.array_equal(out.cpu().numpy(), s["sym"])
    # idempotent: decoding twice gives the same tensor (scripts/test_py_ctx_multiple_get.py:22-30)
    out2 = torch.zeros_like(out)
    fn(_dev(s["payload"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["dec"]), out2, H, D)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("is_k", [True, False])
def test_entropy_encode_matches_oracle(shape, is_k):
    T, B, H, D = shape
    x = S.synth_k(T, B, H, D) if is_k else S.synth_v(T, B, H, D)
    bs = 64 if is_k else 128
    s = _make_stream(x, is_k, 0.1, O.MASK_K_BLOCK if is_k else O.MASK_V_TOKEN, bs)
    m = kc()
    sym = _dev(s["sym"])
    sizes = m.calculate_buffer_size(sym, is_k, H, D)
    assert sizes[0] == s["bi"].size and sizes[1] == s["ti"].size and sizes[2] == 8 and sizes[3] == s["sym"].size
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    fn = m.k_entropy_encode_cuda_export if is_k else m.v_entropy_encode_cuda_export
    base = 12345
    enc, bi, ti = fn(sym, _dev(s["enc"]), bufs[0], bufs[1], bufs[2], bufs[3], base, H, D)
    ref_payload, ref_bi, ref_ti = O.encode_tiles(s["sym"], is_k, s["enc"], base, vec_len=D if is_k else 128)
    assert enc.numel() == ref_payload.size
    assert np.array_equal(ti.cpu().numpy(), ref_ti)
    assert np.array_equal(bi.cpu().numpy(), ref_bi)
    assert np.array_equal(enc.cpu().numpy(), ref_payload)
    idx = bufs[2].cpu().numpy().view(np.uint32)
    assert idx[0] == ref_bi.size // 8 and idx[1] == ref_payload.size


@pytest.mark.parametrize("shape,rep", [((256, 1, 4, 128), 1), ((128, 2, 2, 128), 1), ((128, 2, 2, 128), 4), ((256, 1, 3, 64), 2),
                                       ((256, 2, 2, 96), 1), ((128, 1, 2, 96), 8)])
@pytest.mark.parametrize("mask", [O.MASK_K_BLOCK, O.MASK_CHANNEL])
def test_fused_k_matches_oracle(shape, rep, mask, fused_mode):
    T, B, H, D = shape
    x = S.synth_k(T, B, H, D)
    s = _make_stream(x, True, 0.1, mask, 64)
    q = S.synth_q(B, H * rep, D)
    ref = O.fused_k(s["sym"].reshape(T, B, H, D), s["mn"], s["scale"], mask, 64, S.np16(q))
    m = kc()
    out = torch.zeros(B, H * rep, T, dtype=torch.float16, device=DEV)
    m.k_decode_and_mat_vec_mul_cuda_export(_dev(s["dec"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["payload"]),
                                           _dev(s["mn"].ravel()), _dev(s["scale"].ravel().view(np.uint16), torch.float16),
                                           q.to(DEV), out, H, D)
    got = out.float().cpu().numpy().astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()
    # and against an fp32 PyTorch matmul over the dequantized cache
    deq = torch.from_numpy(O.dequant(s["sym"], s["mn"], s["scale"], mask)).reshape(T, B, H, D).float()
    deq = deq.repeat_interleave(rep, dim=2)
    ref32 = torch.einsum("tbhd,bhd->bht", deq, q.float()).numpy()
    assert np.abs(got - ref32).max() <= 1e-3 * np.abs(ref32).max()


@pytest.mark.parametrize("shape,rep", [((256, 1, 4, 128), 1), ((256, 2, 2, 128), 1), ((256, 2, 2, 128), 4), ((128, 1, 3, 64), 2),
                                       ((256, 2, 2, 96), 1), ((128, 2, 4, 96), 2), ((128, 1, 2, 96), 8)])
@pytest.mark.parametrize("mask", [O.MASK_V_TOKEN, O.MASK_SIM_TOKEN, O.MASK_VECTOR])
def test_fused_v_matches_oracle(shape, rep, mask, fused_mode):
    T, B, H, D = shape
    x = S.synth_v(T, B, H, D)
    s = _make_stream(x, False, 0.2, mask, 128)
    p = S.synth_p(B, H * rep, T)
    ref = O.fused_v(s["sym"].reshape(T, B, H, D), s["mn"], s["scale"], mask, 128, S.np16(p))
    m = kc()
    part = torch.zeros(T // 128, B, H * rep, D, dtype=torch.float16, device=DEV)
    m.v_decode_and_mat_vec_mul_cuda_export(_dev(s["dec"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["payload"]),
                                           _dev(s["mn"].ravel()), _dev(s["scale"].ravel().view(np.uint16), torch.float16),
                                           p.to(DEV), part, H, D)
    got = part.float().sum(dim=0).cpu().numpy().astype(np.float64)     # models/cache/kvcomp_encode.py:275
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()
    deq = torch.from_numpy(O.dequant(s["sym"], s["mn"], s["scale"], mask)).reshape(T, B, H, D).float()
    deq = deq.repeat_interleave(rep, dim=2)
    ref32 = torch.einsum("tbhd,bht->bhd", deq, p.float()).numpy()
    assert np.abs(got - ref32).max() <= 1e-3 * np.abs(ref32).max()


@pytest.mark.parametrize("mask", [O.MASK_K_BLOCK, O.MASK_V_TOKEN, O.MASK_CHANNEL, O.MASK_SIM_TOKEN, O.MASK_VECTOR, O.MASK_SIM_BLOCK])
@pytest.mark.parametrize("eb", [0.03, 0.1, 0.13, 0.2])
def test_quant_dequant_bit_exact(mask, eb):
    _quant_dequant_case(mask, eb)


@pytest.mark.parametrize("eb_k,eb_v", [(0.3, 0.45), (0.03, 0.05)])
def test_fused_across_code_length_regimes(eb_k, eb_v, fused_mode):
    """Short codes (8 symbols per window), and long codes (4 per window with the overflow check)."""
    m = kc()
    T, B, H, D = 256, 1, 4, 128
    s = _make_stream(S.synth_k(T, B, H, D), True, eb_k, O.MASK_CHANNEL, 64)
    q = S.synth_q(B, H, D)
    ref = O.fused_k(s["sym"].reshape(T, B, H, D), s["mn"], s["scale"], O.MASK_CHANNEL, 64, S.np16(q))
    out = torch.zeros(B, H, T, dtype=torch.float16, device=DEV)
    m.k_decode_and_mat_vec_mul_cuda_export(_dev(s["dec"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["payload"]),
                                           _dev(s["mn"].ravel()), _dev(s["scale"].ravel().view(np.uint16), torch.float16),
                                           q.to(DEV), out, H, D)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()
    print("K lmax", int(s["length"].max()))
    s = _make_stream(S.synth_v(T, B, H, D), False, eb_v, O.MASK_V_TOKEN, 128)
    p = S.synth_p(B, H, T)
    ref = O.fused_v(s["sym"].reshape(T, B, H, D), s["mn"], s["scale"], O.MASK_V_TOKEN, 128, S.np16(p))
    part = torch.zeros(T // 128, B, H, D, dtype=torch.float16, device=DEV)
    m.v_decode_and_mat_vec_mul_cuda_export(_dev(s["dec"]), _dev(s["bi"]), _dev(s["ti"]), _dev(s["payload"]),
                                           _dev(s["mn"].ravel()), _dev(s["scale"].ravel().view(np.uint16), torch.float16),
                                           p.to(DEV), part, H, D)
    assert np.abs(part.float().sum(0).cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()
    print("V lmax", int(s["length"].max()))


@pytest.mark.parametrize("mask", [O.MASK_V_TOKEN, O.MASK_CHANNEL, O.MASK_SIM_TOKEN, O.MASK_VECTOR])
def test_quant_narrow_rows_bit_exact(mask):
    """Rows whose length is not a multiple of 8 take the quantizer's two-elements-per-lane kernels instead of the
    eight-per-lane ones."""
    _quant_dequant_case(mask, 0.1, geometry=(128, 1, 3, 6))


@pytest.mark.parametrize("geometry", [(128, 1, 48, 128), (128, 3, 4, 72), (64, 1, 96, 128), (64, 1, 100, 128), (64, 1, 130, 128)])
def test_quant_rows_kept_in_registers_bit_exact(geometry):
    """Per-token rows of 512 to 16 384 elements are read once and kept in the wave's registers (8, 16, 24 or 32 chunks
    of 16 bytes per lane: rows of 6144, 864 -- whose last chunk only some lanes hold --, 12 288 and 12 800 elements),
    longer ones (16 640) are read twice; per-channel blocks of 64 tokens are kept in registers at any width."""
    for mask in (O.MASK_V_TOKEN, O.MASK_CHANNEL):
        _quant_dequant_case(mask, 0.1, geometry=geometry)


def _quant_dequant_case(mask, eb, geometry=(256, 2, 4, 128)):
    from kvcomp_amd import compute as cp
    T, B, H, D = geometry
    x = S.synth_k(T, B, H, D)
    x5 = S.blocked(x, 64)
    _, _, scale, sym, mn = O.quant(S.np16(x5), mask, eb)
    dims = [i + 1 for i in range(4) if mask & (1 << i)]
    counts = torch.zeros(256, dtype=torch.int64, device=DEV)
    g_sym, g_min, g_scale = cp.quant(x5.to(DEV), dims, eb, counts=counts)
    assert tuple(g_scale.shape) == scale.shape
    assert np.array_equal(g_scale.cpu().numpy().view(np.uint16), scale.view(np.uint16))
    assert np.array_equal(g_min.cpu().numpy(), mn)
    assert np.array_equal(g_sym.cpu().numpy(), sym)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(sym.ravel(), minlength=256))
    deq = cp.dequant(g_sym, g_min, g_scale, dims)
    assert np.array_equal(deq.cpu().numpy().view(np.uint16), O.dequant(sym, mn, scale, mask).view(np.uint16))
    assert O.check_error_bound(S.np16(x5), deq.cpu().numpy(), scale, mask) == 0


def test_quant_matches_torch_fp16_ops_on_device():
    """The same op chain as utils/compute.py:93-106, run by stock PyTorch on the GPU, gives the same bits."""
    from kvcomp_amd import compute as cp
    x5 = S.blocked(S.synth_k(128, 1, 4, 128), 64).to(DEV)
    for dims, eb in (([1, 2, 3, 4], 0.1), ([2, 3, 4], 0.07), ([1], 0.13)):
        mn, mx = x5, x5
        for d in dims:
            mn = mn.min(dim=d, keepdim=True).values
            mx = mx.max(dim=d, keepdim=True).values
        sc = (mx - mn) * eb
        mi = (mn / sc).round_()
        qi = (x5 / sc).round_() - mi
        g_sym, g_min, g_scale = cp.quant(x5, dims, eb)
        assert torch.equal(g_scale, sc)
        assert torch.equal(g_min, mi.to(torch.int8))
        assert torch.equal(g_sym, qi.to(torch.uint8))


def test_build_codebook_matches_oracle():
    m = kc()
    x5 = S.np16(S.blocked(S.synth_k(256, 1, 4, 128), 64))
    sym = O.quant(x5, O.MASK_K_BLOCK, 0.05)[3]
    shift, enc, dec = m.build_codebook([_dev(sym[:2]), _dev(sym[2:])])
    r_shift, r_enc, r_dec = O.build_codebook(sym)
    assert shift == r_shift == 0
    assert enc.device.type == "cpu" and dec.device.type == "cpu"
    assert np.array_equal(enc.numpy(), r_enc)
    assert np.array_equal(dec.numpy(), r_dec)


def _skewed_symbols(shape, nsym, rng):
    """Fibonacci counts (1, 1, 2, 3, 5, ...): the Huffman code degenerates to lengths up to nsym - 1."""
    fib = [1, 1]
    while len(fib) < nsym:
        fib.append(fib[-1] + fib[-2])
    n = int(np.prod(shape))
    assert sum(fib) <= n
    flat = np.concatenate([np.full(c, k, np.uint8) for k, c in enumerate(fib)] + [np.full(n - sum(fib), nsym - 1, np.uint8)])
    rng.shuffle(flat)
    return flat.reshape(shape)


@pytest.mark.parametrize("is_k", [True, False])
@pytest.mark.parametrize("nsym", [14, 22])
def test_long_codes_take_the_spill_path(is_k, nsym):
    """Codes longer than the 10-bit table index (and, for 24 symbols, longer than 16 bits)."""
    rng = np.random.default_rng(5)
    T, B, H, D = 256, 1, 2, 128
    sym = _skewed_symbols((T // (64 if is_k else 128), 64 if is_k else 128, B, H, D), nsym, rng)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts)
    assert length.max() == nsym - 1
    _, enc = O.encode_table(code, length, counts)
    st, dec = O.decode_tree(code, length, counts)
    assert st == 0
    payload, bi, ti = O.encode_tiles(sym, is_k, enc, 0)
    m = kc()
    out = torch.zeros(sym.shape, dtype=torch.uint8, device=DEV)
    fn = m.k_entropy_decode_cuda_export if is_k else m.v_entropy_decode_cuda_export
    fn(_dev(payload), _dev(bi), _dev(ti), _dev(dec), out, H, D)
    assert np.array_equal(out.cpu().numpy(), sym)
    sizes = m.calculate_buffer_size(_dev(sym), is_k, H, D)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    efn = m.k_entropy_encode_cuda_export if is_k else m.v_entropy_encode_cuda_export
    g_enc, g_bi, g_ti = efn(_dev(sym), _dev(enc), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
    assert np.array_equal(g_enc.cpu().numpy(), payload)
    assert np.array_equal(g_ti.cpu().numpy(), ti) and np.array_equal(g_bi.cpu().numpy(), bi)


def test_wide_alphabet_uses_int16_tree():
    """More than 64 symbols cannot be expressed in the reference's int8 tree; the wide tree decodes them."""
    m = kc()
    x5 = S.blocked(S.synth_v(256, 1, 2, 128), 128)
    sym = O.quant(S.np16(x5), O.MASK_V_TOKEN, 0.004)[3]
    assert len(np.unique(sym)) > 64
    d_sym = _dev(sym)
    with pytest.raises(RuntimeError):
        m.build_codebook([d_sym])
    shift, enc, dec = m.build_codebook([d_sym], tree_format=m.TREE_I16)
    assert shift == 0
    sizes = m.calculate_buffer_size(d_sym, False, 2, 128)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    g_enc, g_bi, g_ti = m.v_entropy_encode_cuda_export(d_sym, enc.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, 2, 128)
    ref_payload, ref_bi, ref_ti = O.encode_tiles(sym, False, enc.numpy(), 0)
    assert np.array_equal(g_enc.cpu().numpy(), ref_payload)
    out = torch.zeros_like(d_sym)
    m.v_entropy_decode_cuda_export(g_enc, g_bi, g_ti, dec.to(DEV), out, 2, 128, tree_format=m.TREE_I16)
    assert torch.equal(out, d_sym)


def test_k_mat_vec_mul_dense():
    m = kc()
    T, B, H, D = 512, 2, 4, 128
    k = S.synth_k(T, B, H, D).to(DEV)
    q = S.synth_q(B, H, D).to(DEV)
    out = torch.zeros(T, B, H, dtype=torch.float16, device=DEV)
    ms = m.k_mat_vec_mul_cuda_export(k, q, out)
    ref = torch.einsum("tbhd,bhd->tbh", k.float(), q.float())
    assert ms >= 0
    assert (out.float() - ref).abs().max() <= 1e-3 * ref.abs().max()


def test_errors_raise_instead_of_aborting():
    m = kc()
    sym = torch.zeros(1, 60, 1, 1, 128, dtype=torch.uint8, device=DEV)      # 60 tokens: not a multiple of 64
    with pytest.raises(RuntimeError):
        m.calculate_buffer_size(sym, True, 1, 128)
    with pytest.raises(RuntimeError):
        m.build_codebook([torch.zeros(100, dtype=torch.uint8, device=DEV)])   # a lone symbol has no usable code


@pytest.mark.parametrize("binding", ["ctypes", "compiled"])
@pytest.mark.parametrize("is_k", [True, False])
def test_empty_inputs_are_no_ops(is_k, binding):
    """Zero tokens: sizes are zero, the encoder returns empty views, the decoders and the fused products return without
    touching anything (the reference would launch an empty grid and abort on the launch error)."""
    if binding == "ctypes":
        m = kc()
    else:
        import importlib.util
        from kvcomp_amd import build
        spec = importlib.util.spec_from_file_location("kvcomp_cuda", build.MODULE_PATH)
        m = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(m)
    H, D = 4, 128
    bs = 64 if is_k else 128
    x = S.synth_k(128, 1, H, D)
    sym = _make_stream(x, True, 0.1, O.MASK_K_BLOCK, 64)["sym"]
    _, enc, tree = m.build_codebook([_dev(sym)])
    empty = torch.zeros(0, bs, 1, H, D, dtype=torch.uint8, device=DEV)
    assert tuple(m.calculate_buffer_size(empty, is_k, H, D)) == (0, 0, 8, 0)
    bufs = [torch.full((8,), 0xAB, dtype=torch.uint8, device=DEV) for _ in range(4)]
    efn = m.k_entropy_encode_cuda_export if is_k else m.v_entropy_encode_cuda_export
    payload, bi, ti = efn(empty, enc.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
    assert payload.numel() == bi.numel() == ti.numel() == 0
    assert all(bool((b == 0xAB).all()) for b in (bufs[0], bufs[1], bufs[3]))
    z = torch.zeros(0, dtype=torch.uint8, device=DEV)
    dfn = m.k_entropy_decode_cuda_export if is_k else m.v_entropy_decode_cuda_export
    assert dfn(z, z, z, tree.to(DEV), empty, H, D) == 0.0
    mins, scales = torch.zeros(0, dtype=torch.int8, device=DEV), torch.zeros(0, dtype=torch.float16, device=DEV)
    if is_k:
        out = torch.zeros(1, H, 0, dtype=torch.float16, device=DEV)
        assert m.k_decode_and_mat_vec_mul_cuda_export(tree.to(DEV), z, z, z, mins, scales, S.synth_q(1, H, D).to(DEV), out, H, D) == 0.0
    else:
        p = torch.zeros(1, H, 0, dtype=torch.float16, device=DEV)
        out = torch.zeros(0, 1, H, D, dtype=torch.float16, device=DEV)
        assert m.v_decode_and_mat_vec_mul_cuda_export(tree.to(DEV), z, z, z, mins, scales, p, out, H, D) == 0.0
    torch.cuda.synchronize()


@pytest.mark.parametrize("is_k", [True, False])
@pytest.mark.parametrize("nsym", [14, 22])
def test_fused_with_long_codes_uses_slow_path(is_k, nsym, fused_mode):
    """Codebooks whose codes exceed the table index: the fused kernels must fall back and still be right."""
    rng = np.random.default_rng(8)
    T, B, H, D = 256, 1, 2, 128
    bs = 64 if is_k else 128
    sym = _skewed_symbols((T // bs, bs, B, H, D), nsym, rng)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    code, length = O.huffman_build(counts)
    _, enc = O.encode_table(code, length, counts)
    st, dec = O.decode_tree(code, length, counts)
    payload, bi, ti = O.encode_tiles(sym, is_k, enc, 0)
    mask = O.MASK_K_BLOCK if is_k else O.MASK_V_TOKEN
    gs = O.group_shape(sym.shape, mask)
    mn = rng.integers(-20, 5, size=gs).astype(np.int8)
    scale = rng.uniform(0.05, 0.5, size=gs).astype(np.float16)
    m = kc()
    args = (_dev(dec), _dev(bi), _dev(ti), _dev(payload), _dev(mn.ravel()), _dev(scale.ravel().view(np.uint16), torch.float16))
    if is_k:
        q = S.synth_q(B, H, D)
        ref = O.fused_k(sym.reshape(T, B, H, D), mn, scale, mask, bs, S.np16(q))
        out = torch.zeros(B, H, T, dtype=torch.float16, device=DEV)
        m.k_decode_and_mat_vec_mul_cuda_export(*args, q.to(DEV), out, H, D)
        got = out.float().cpu().numpy()
    else:
        p = S.synth_p(B, H, T)
        ref = O.fused_v(sym.reshape(T, B, H, D), mn, scale, mask, bs, S.np16(p))
        part = torch.zeros(T // 128, B, H, D, dtype=torch.float16, device=DEV)
        m.v_decode_and_mat_vec_mul_cuda_export(*args, p.to(DEV), part, H, D)
        got = part.float().sum(0).cpu().numpy()
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()


@pytest.mark.parametrize("nsym,expect_lmax", [(200, 8), (12, 4), (7, 3)])
def test_fused_k_window_groupings(nsym, expect_lmax, fused_mode):
    """Near-uniform alphabets pin the code length, hence which window grouping the fused kernel takes:
    200 symbols -> 8-bit codes, too dense for four per window (two per refill); 12 -> 4-bit codes (four per
    refill, guaranteed); 7 -> 3-bit codes (eight per refill).  The 200-symbol book needs the int16 tree."""
    rng = np.random.default_rng(21)
    m = kc()
    T, B, H, D = 128, 1, 2, 64
    sym = rng.integers(0, nsym, size=(T // 64, 64, B, H, D)).astype(np.uint8)
    fmt = m.TREE_I16 if nsym > 64 else m.TREE_I8
    shift, enc, dec = m.build_codebook([_dev(sym)], tree_format=fmt)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    assert int(O.huffman_build(counts)[1].max()) == expect_lmax
    sizes = m.calculate_buffer_size(_dev(sym), True, H, D)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    g_enc, g_bi, g_ti = m.k_entropy_encode_cuda_export(_dev(sym), enc.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
    ref_payload, _, _ = O.encode_tiles(sym, True, enc.numpy(), 0, vec_len=D)
    assert np.array_equal(g_enc.cpu().numpy(), ref_payload)
    gs = O.group_shape(sym.shape, O.MASK_CHANNEL)
    mn = rng.integers(-(nsym // 2) - 1, 0, size=gs).astype(np.int8)       # symbols centred on zero, like real groups
    scale = rng.uniform(0.01, 0.2, size=gs).astype(np.float16)
    q = S.synth_q(B, H, D)
    ref = O.fused_k(sym.reshape(T, B, H, D), mn, scale, O.MASK_CHANNEL, 64, S.np16(q))
    out = torch.zeros(B, H, T, dtype=torch.float16, device=DEV)
    m.k_decode_and_mat_vec_mul_cuda_export(dec.to(DEV), g_bi, g_ti, g_enc, _dev(mn.ravel()),
                                           _dev(scale.ravel().view(np.uint16), torch.float16), q.to(DEV), out, H, D,
                                           tree_format=fmt)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()


@pytest.mark.parametrize("D,rep", [(64, 1), (96, 1), (128, 1), (72, 1), (128, 4), (96, 2), (64, 8)])
@pytest.mark.parametrize("nsym,expect_lmax", [(12, 4), (24, 5), (40, 6), (100, 7)])
def test_fused_group_sizes_and_remainders(nsym, expect_lmax, D, rep, fused_mode):
    """Exactly uniform alphabets give codes of 4 to 7 bits, for which a 30-bit half window is sure to hold 7, 6, 5
    and 4 symbols: the kernel decodes 14, 12, 10 or 8 symbols per refill and finishes a vector whose length is not
    a multiple of that with refills of 8 (head_dim 64, 72, 96 and 128; V vectors hold 128 symbols)."""
    rng = np.random.default_rng(100 * nsym + D)
    m = kc()
    T, B, H = 128, 1, 2
    sym = (rng.permutation(T * B * H * D) % nsym).astype(np.uint8).reshape(T // 64, 64, B, H, D)
    fmt = m.TREE_I16 if nsym > 64 else m.TREE_I8
    shift, enc, dec = m.build_codebook([_dev(sym)], tree_format=fmt)
    counts = np.bincount(sym.ravel(), minlength=256).astype(np.int64)
    assert int(O.huffman_build(counts)[1].max()) == expect_lmax
    # K: one scale / minimum per channel of each 64-token block
    sizes = m.calculate_buffer_size(_dev(sym), True, H, D)
    bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
    g_enc, g_bi, g_ti = m.k_entropy_encode_cuda_export(_dev(sym), enc.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
    gs = O.group_shape(sym.shape, O.MASK_CHANNEL)
    mn = rng.integers(-(nsym // 2) - 1, 0, size=gs).astype(np.int8)
    scale = rng.uniform(0.01, 0.2, size=gs).astype(np.float16)
    q = S.synth_q(B, H * rep, D)
    ref = O.fused_k(sym.reshape(T, B, H, D), mn, scale, O.MASK_CHANNEL, 64, S.np16(q))
    out = torch.zeros(B, H * rep, T, dtype=torch.float16, device=DEV)
    m.k_decode_and_mat_vec_mul_cuda_export(dec.to(DEV), g_bi, g_ti, g_enc, _dev(mn.ravel()),
                                           _dev(scale.ravel().view(np.uint16), torch.float16), q.to(DEV), out, H, D,
                                           tree_format=fmt)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()
    # V: one scale / minimum per token
    if (B * H * D) % 64 == 0:
        symv = sym.reshape(T // 128, 128, B, H, D)
        sizes = m.calculate_buffer_size(_dev(symv), False, H, D)
        bufs = [torch.zeros(n, dtype=torch.uint8, device=DEV) for n in sizes]
        v_enc, v_bi, v_ti = m.v_entropy_encode_cuda_export(_dev(symv), enc.to(DEV), bufs[0], bufs[1], bufs[2], bufs[3], 0, H, D)
        gsv = O.group_shape(symv.shape, O.MASK_V_TOKEN)
        mnv = rng.integers(-(nsym // 2) - 1, 0, size=gsv).astype(np.int8)
        scv = rng.uniform(0.01, 0.2, size=gsv).astype(np.float16)
        p = S.synth_p(B, H * rep, T)
        refv = O.fused_v(symv.reshape(T, B, H, D), mnv, scv, O.MASK_V_TOKEN, 128, S.np16(p))
        part = torch.zeros(T // 128, B, H * rep, D, dtype=torch.float16, device=DEV)
        m.v_decode_and_mat_vec_mul_cuda_export(dec.to(DEV), v_bi, v_ti, v_enc, _dev(mnv.ravel()),
                                               _dev(scv.ravel().view(np.uint16), torch.float16), p.to(DEV), part, H, D,
                                               tree_format=fmt)
        got = part.float().sum(0).cpu().numpy()
        assert np.abs(got - refv).max() <= 1e-3 * np.abs(refv).max()
