"""Pins of the oracle's fp16 conversions and quantizer (Q1-Q3) that do not rest on the oracle's own formula:
numpy's float16 conversions, stock PyTorch CPU fp16 ops (library routines), closed forms, invariants, and --
where it was built -- the reference's own C++ quant compiled into oracle/_ref."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import ref as R
from tests import _synth as S

MASK_DIMS = {O.MASK_K_BLOCK: [1, 2, 3, 4], O.MASK_V_TOKEN: [2, 3, 4], O.MASK_CHANNEL: [1],
             O.MASK_SIM_TOKEN: [3, 4], O.MASK_VECTOR: [4], O.MASK_SIM_BLOCK: [1, 3, 4]}


def test_h2f_exhaustive_against_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    mine = np.array([O.h2f(int(h)) for h in allh], dtype=np.float32)
    same = (ref.view(np.uint32) == mine.view(np.uint32)) | (np.isnan(ref) & np.isnan(mine))
    assert same.all()


def test_f2h_against_numpy_including_ties_and_boundaries():
    rng = np.random.default_rng(0)
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    fin = np.sort(halves[np.isfinite(halves)])
    mids = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)   # exact ties
    vals = [fin, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
            np.array([65519.996, 65520.0, 65536.0, 1e9, -1e9, 2.9802322e-08, 2.9802326e-08, 5.9604645e-08, 1e-10, 0.0, -0.0],
                     np.float32)]
    vals += [(rng.standard_normal(4000) * s).astype(np.float32) for s in (1e-8, 1e-6, 1e-4, 1e-2, 1.0, 100.0, 30000.0)]
    vals = np.concatenate(vals)
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).view(np.uint16)
    mine = np.array([O.f2h(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(ref, mine)


def _torch_quant(x5, dims, eb):
    """utils/compute.py:93-106 spelled with stock PyTorch ops (the library, not the reference code)."""
    mn, mx = x5, x5
    for d in dims:
        mn = mn.min(dim=d, keepdim=True).values
        mx = mx.max(dim=d, keepdim=True).values
    sc = (mx - mn) * eb
    mi = (mn / sc).round()
    qi = (x5 / sc).round() - mi
    return qi, mi, sc


@pytest.mark.parametrize("mask", sorted(MASK_DIMS))
@pytest.mark.parametrize("eb", [0.03, 0.05, 0.1, 0.13, 0.2, 0.3])
def test_quant_bit_exact_against_torch_cpu_fp16_ops(mask, eb):
    x5 = S.blocked(S.synth_k(192, 2, 3, 128), 64)
    qi, mi, sc = _torch_quant(x5, MASK_DIMS[mask], eb)
    s16, m16, c16, s8, m8 = O.quant(x5.numpy(), mask, eb)
    assert np.array_equal(sc.numpy().view(np.uint16), c16.view(np.uint16))
    assert np.array_equal(mi.numpy().view(np.uint16), m16.view(np.uint16))
    assert np.array_equal(qi.numpy().view(np.uint16), s16.view(np.uint16))
    assert np.array_equal(qi.to(torch.uint8).numpy(), s8)
    assert np.array_equal(mi.to(torch.int8).numpy(), m8)
    # Q2: (uint8 + int8) * fp16, exactly as models/cache/kvcomp_encode.py:146 computes it
    deq = (qi.to(torch.uint8) + mi.to(torch.int8)) * sc
    mine = O.dequant(s8, m8, c16, mask)
    assert np.array_equal(deq.numpy().view(np.uint16), mine.view(np.uint16))
    # invariants: smallest symbol of every group is 0; alphabet <= ceil(1/eb) + 2; Q3 bound
    assert s8.min() == 0 and int(s8.max()) <= int(np.ceil(1 / eb)) + 2
    assert O.check_error_bound(x5.numpy(), mine, c16, mask) == 0


def test_quant_laplace_heavy_tail_against_torch():
    x5 = S.blocked(S.synth_laplace(128, 1, 2, 96, 11), 64)
    for mask, eb in ((O.MASK_CHANNEL, 0.05), (O.MASK_V_TOKEN, 0.3), (O.MASK_K_BLOCK, 0.2)):
        qi, mi, sc = _torch_quant(x5, MASK_DIMS[mask], eb)
        s16, m16, c16, s8, m8 = O.quant(x5.numpy(), mask, eb)
        assert np.array_equal(qi.numpy().view(np.uint16), s16.view(np.uint16))
        assert np.array_equal(sc.numpy().view(np.uint16), c16.view(np.uint16))


def test_quant_brute_force_every_fp16_in_a_range():
    """One group that holds every fp16 value in [-3, 5]: the double rounding (f32 divide -> fp16 -> half-even
    round -> fp16 subtract) is compared element by element with PyTorch."""
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    vals = halves[np.isfinite(halves) & (halves >= -3) & (halves <= 5)]
    n = 64 * 8 * 128
    assert vals.size <= n
    buf = np.full(n, 5.0, np.float16)
    buf[:vals.size] = vals
    x5 = torch.from_numpy(buf.reshape(1, 64, 1, 8, 128))
    for eb in (0.03, 0.1, 0.13, 0.3):
        qi, mi, sc = _torch_quant(x5, [1, 2, 3, 4], eb)
        s16, m16, c16, s8, m8 = O.quant(x5.numpy(), O.MASK_K_BLOCK, eb)
        assert np.array_equal(qi.numpy().view(np.uint16), s16.view(np.uint16))
        assert np.array_equal(mi.numpy().view(np.uint16), m16.view(np.uint16))


def test_quant_closed_form_small_case():
    """min 0, max 5, eb 0.1 -> scale 0.5 exactly, min_i 0, sym = round_half_even(x / 0.5)."""
    x = np.zeros((1, 64, 1, 1, 2), np.float16)
    xs = np.array([0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 2.26, 4.74, 5.0], np.float16)
    x.reshape(-1)[:xs.size] = xs
    s16, m16, c16, s8, m8 = O.quant(x, O.MASK_K_BLOCK, 0.1)
    assert float(c16.ravel()[0]) == 0.5 and int(m8.ravel()[0]) == 0
    assert s8.reshape(-1)[:xs.size].tolist() == [0, 0, 1, 2, 2, 2, 5, 9, 10]     # 0.5 -> 0 and 2.5 -> 2: ties to even
    # shifting every value by -2 (= -4 steps, an even count, so ties keep their parity) moves min_i to -4 only
    s16b, m16b, c16b, s8b, m8b = O.quant((x.astype(np.float32) - 2.0).astype(np.float16), O.MASK_K_BLOCK, 0.1)
    assert int(m8b.ravel()[0]) == -4 and np.array_equal(s8b, s8)
    # dequant closed form
    d = O.dequant(s8b, m8b, c16b, O.MASK_K_BLOCK)
    assert np.array_equal(d.reshape(-1)[:xs.size].astype(np.float32), (np.array([0, 0, 1, 2, 2, 2, 5, 9, 10]) - 4) * 0.5)


def test_dequant_brute_force_against_torch():
    ints = np.arange(-128, 383, dtype=np.int32)
    rng = np.random.default_rng(3)
    scales = np.concatenate([rng.uniform(1e-4, 4.0, 40), [6.1e-5, 1e-7, 0.5, 1.0]]).astype(np.float16)
    for sc in scales:
        ref = (torch.from_numpy(ints.astype(np.int16)) * torch.tensor(sc, dtype=torch.float16).reshape(1)).numpy()
        mine = np.array([O.f2h(float(i) * O.h2f(int(np.float16(sc).view(np.uint16)))) for i in ints], np.uint16)
        assert np.array_equal(ref.view(np.uint16), mine)


@pytest.mark.skipif(not R.available(), reason="oracle/_ref (reference C++ built in place) not present")
@pytest.mark.parametrize("mask", [O.MASK_K_BLOCK, O.MASK_V_TOKEN, O.MASK_CHANNEL, O.MASK_VECTOR])
def test_quant_against_reference_cpp(mask):
    x5 = S.blocked(S.synth_k(128, 2, 2, 128), 64).numpy()
    a = R.quant(x5, MASK_DIMS[mask], 0.1)
    b = O.quant(x5, mask, 0.1)
    for i in range(3):
        assert np.array_equal(a[i].view(np.uint16).ravel(), b[i].view(np.uint16).ravel())


def test_blocks_to_compress_table():
    """C1: n = (len + bs - len % bs - recent) // bs  (utils/compute.py:51-52)."""
    bs = 64
    for recent in (bs, 2 * bs, 4 * bs):
        for length in range(0, 4 * bs + 1):
            n = O.blocks_to_compress(length, bs, recent)
            assert n == (length // bs) + 1 - recent // bs     # closed form for recent a multiple of bs
            if R.available() and length % 17 == 0:
                assert R.cut_rows(0, length, bs, recent) == max(0, n) * bs
