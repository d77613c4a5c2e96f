"""numpy front end of the CPU oracle (oracle/kvc_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module; the product
(kvcomp_amd) never does.  Each wrapper names the reference file:line its C function restates.
"""
import ctypes as C
import heapq
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

# reduce masks over (BS=1, B=2, H=4, D=8) of the [NB, BS, B, H, D] layout
MASK_K_BLOCK = 0xF      # models/cache/kvcomp_encode.py:10-13  BlockQuant dims [1,2,3,4]
MASK_V_TOKEN = 0xE      # models/cache/kvcomp_encode.py:10-13  TokenQuant dims [2,3,4]
MASK_CHANNEL = 0x1      # utils/compute.py:140  ChannelQuant (per b, h, block, channel)
MASK_SIM_TOKEN = 0xC    # utils/compute.py:141  TokenQuant of the sim path (per b, block, token)
MASK_VECTOR = 0x8       # utils/compute.py:142  VectorQuant
MASK_SIM_BLOCK = 0xD    # utils/compute.py:139  BlockQuant of the sim path (per b, block)

VEC_PER_TILE = 64


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libkvc_oracle.so")
        if not os.path.exists(path):
            import subprocess
            import sys
            subprocess.check_call([sys.executable, os.path.join(_HERE, "build_oracle.py"), "--no-ref"])
        L = C.CDLL(path)
        L.kvo_h2f.restype = C.c_float
        L.kvo_h2f.argtypes = [C.c_uint16]
        L.kvo_f2h.restype = C.c_uint16
        L.kvo_f2h.argtypes = [C.c_float]
        for name in ("kvo_quant_groups", "kvo_check_error_bound", "kvo_blocks_to_compress", "kvo_encode_table",
                     "kvo_decode_tree", "kvo_huffman_bits", "kvo_tile_count", "kvo_encode_tiles",
                     "kvo_decode_tiles", "kvo_fused_k_from_stream"):
            getattr(L, name).restype = C.c_int64
        _LIB = L
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(v):
    return C.c_int64(int(v))


def h2f(h):
    return lib().kvo_h2f(int(h))


def f2h(f):
    return lib().kvo_f2h(C.c_float(float(f)))


def quant_groups(shape5, mask):
    NB, BS, B, H, D = shape5
    return int(lib().kvo_quant_groups(_i64(NB), _i64(BS), _i64(B), _i64(H), _i64(D), C.c_int(mask)))


def group_shape(shape5, mask):
    NB, BS, B, H, D = shape5
    return (NB, 1 if mask & 1 else BS, 1 if mask & 2 else B, 1 if mask & 4 else H, 1 if mask & 8 else D)


def quant(x, mask, eb):
    """Q1: utils/compute.py:93-106 / :74-91.  x float16 [NB,BS,B,H,D].
    Returns (sym_f16, min_f16, scale_f16, sym_u8, min_i8); metadata arrays have group_shape()."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    NB, BS, B, H, D = x.shape
    gs = group_shape(x.shape, mask)
    G = int(np.prod(gs))
    sym16 = np.empty(x.shape, np.uint16)
    sym8 = np.empty(x.shape, np.uint8)
    mn16 = np.empty(G, np.uint16)
    sc16 = np.empty(G, np.uint16)
    mn8 = np.empty(G, np.int8)
    rc = lib().kvo_quant(_p(x.view(np.uint16)), _i64(NB), _i64(BS), _i64(B), _i64(H), _i64(D), C.c_int(mask),
                         C.c_float(eb), _p(sym16), _p(mn16), _p(sc16), _p(sym8), _p(mn8))
    assert rc == 0
    return (sym16.view(np.float16), mn16.view(np.float16).reshape(gs), sc16.view(np.float16).reshape(gs),
            sym8, mn8.reshape(gs))


def dequant(sym_u8, min_i8, scale_f16, mask):
    """Q2: models/cache/kvcomp_encode.py:146."""
    sym_u8 = np.ascontiguousarray(sym_u8, dtype=np.uint8)
    NB, BS, B, H, D = sym_u8.shape
    out = np.empty(sym_u8.shape, np.uint16)
    mn = np.ascontiguousarray(min_i8, dtype=np.int8).ravel()
    sc = np.ascontiguousarray(scale_f16, dtype=np.float16).ravel()
    lib().kvo_dequant(_p(sym_u8), _p(mn), _p(sc.view(np.uint16)), _i64(NB), _i64(BS), _i64(B), _i64(H), _i64(D),
                      C.c_int(mask), _p(out))
    return out.view(np.float16)


def check_error_bound(x, xhat, scale_f16, mask):
    """Q3: src/compute.cpp:60-69.  Number of elements violating |x - xhat| < 0.53*scale."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    xhat = np.ascontiguousarray(xhat, dtype=np.float16)
    NB, BS, B, H, D = x.shape
    sc = np.ascontiguousarray(scale_f16, dtype=np.float16).ravel()
    return int(lib().kvo_check_error_bound(_p(x.view(np.uint16)), _p(xhat.view(np.uint16)), _p(sc.view(np.uint16)),
                                           _i64(NB), _i64(BS), _i64(B), _i64(H), _i64(D), C.c_int(mask)))


def blocks_to_compress(length, block_size, recent_size):
    """C1: utils/compute.py:59-72."""
    return int(lib().kvo_blocks_to_compress(_i64(length), _i64(block_size), _i64(recent_size)))


def huffman_build(counts, h2_single=False):
    """H1/H2: src/huffman.cpp:34-96, utils/huffman.py:46-81.  Returns (code u32[n], length u32[n])."""
    counts = np.ascontiguousarray(counts, dtype=np.int64)
    n = counts.shape[0]
    code = np.zeros(n, np.uint32)
    length = np.zeros(n, np.uint32)
    rc = lib().kvo_huffman_build(_p(counts), C.c_int(n), C.c_int(1 if h2_single else 0), _p(code), _p(length))
    if rc < 0:
        raise ValueError("a Huffman code exceeds 32 bits")
    return code, length


def encode_table(code, length, counts):
    """T1: src/huffman.cpp:166-187.  Returns (shift, uint8 table)."""
    counts = np.ascontiguousarray(counts, dtype=np.int64)
    buf = np.zeros(8 * counts.shape[0], np.uint8)
    shift = C.c_int(0)
    nb = lib().kvo_encode_table(_p(code), _p(length), _p(counts), C.c_int(counts.shape[0]), _p(buf), C.byref(shift))
    return shift.value, buf[:nb].copy()


def decode_tree(code, length, counts, cap_nodes=1024):
    """T2: src/huffman.cpp:229-252.  Returns (status, uint8 tree); status < 0 flags the reference's
    int8 limits (-2) or the lone-symbol case (-3)."""
    counts = np.ascontiguousarray(counts, dtype=np.int64)
    buf = np.zeros(3 * cap_nodes, np.uint8)
    nb = lib().kvo_decode_tree(_p(code), _p(length), _p(counts), C.c_int(counts.shape[0]), _p(buf),
                               _i64(buf.shape[0]))
    if nb >= 0:
        return 0, buf[:nb].copy()
    return int(nb), buf


def build_codebook(symbols):
    """src/huffman.cpp:99-157 on one uint8 array.  Returns (shift, encode_table, decode_tree)."""
    counts = np.bincount(np.asarray(symbols, dtype=np.uint8).ravel(), minlength=256).astype(np.int64)
    code, length = huffman_build(counts)
    shift, enc = encode_table(code, length, counts)
    st, dec = decode_tree(code, length, counts)
    if st < 0:
        raise ValueError("decode tree not representable in the reference format (status %d)" % st)
    return shift, enc, dec


def huffman_bits(symbols, code, length):
    """H2: utils/huffman.py:83-95.  Returns a bool array, one entry per bit."""
    sym = np.ascontiguousarray(symbols, dtype=np.uint8).ravel()
    cap = int(sym.shape[0]) * int(max(1, length.max()))
    bits = np.empty(cap, np.uint8)
    code = np.ascontiguousarray(code, dtype=np.uint32)
    length = np.ascontiguousarray(length, dtype=np.uint32)
    assert code.shape[0] >= 256 and length.shape[0] >= 256
    nb = lib().kvo_huffman_bits(_p(sym), _i64(sym.shape[0]), _p(code), _p(length), _p(bits), _i64(cap))
    assert nb >= 0
    return bits[:nb].astype(bool)


def tile_count(tokens, stride, is_k, vec_len=128):
    return int(lib().kvo_tile_count(_i64(tokens), _i64(stride), C.c_int(int(is_k)), C.c_int(vec_len)))


def encode_tiles(sym5, is_k, table, base_global_offset=0, vec_len=128):
    """E1-E3: src/kernels.cu:181-235,419-596.  sym5 uint8 [NB,BS,B,H,D].
    Returns (payload, block_infos, thread_infos) as uint8 arrays, tiles in tile order."""
    sym5 = np.ascontiguousarray(sym5, dtype=np.uint8)
    NB, BS, B, H, D = sym5.shape
    tokens, stride = NB * BS, B * H * D
    tiles = tile_count(tokens, stride, is_k, vec_len)
    cap = sym5.size * 4 + 64
    payload = np.zeros(cap, np.uint8)
    bi = np.zeros(tiles * 8, np.uint8)
    ti = np.zeros(tiles * VEC_PER_TILE * 2, np.uint8)
    table = np.ascontiguousarray(table, dtype=np.uint8)
    total = lib().kvo_encode_tiles(_p(sym5), _i64(tokens), _i64(stride), C.c_int(int(is_k)), C.c_int(vec_len),
                                   _p(table), _i64(table.shape[0] // 8), C.c_uint32(base_global_offset),
                                   _p(payload), _i64(cap), _p(bi), _p(ti))
    if total < 0:
        raise ValueError("encode_tiles failed (%d)" % total)
    return payload[:total].copy(), bi, ti


def decode_tiles(encoded, block_infos, thread_infos, tree, shape5, is_k, vec_len=128):
    """D1/D2: src/kernels.cu:237-291,598-719.  Returns uint8 [NB,BS,B,H,D]."""
    NB, BS, B, H, D = shape5
    out = np.zeros(shape5, np.uint8)
    enc = np.ascontiguousarray(encoded, dtype=np.uint8)
    tree = np.ascontiguousarray(tree, dtype=np.uint8)
    rc = lib().kvo_decode_tiles(_p(enc), _p(np.ascontiguousarray(block_infos)), _p(np.ascontiguousarray(thread_infos)),
                                _p(tree), _i64(tree.shape[0]), _i64(NB * BS), _i64(B * H * D), C.c_int(int(is_k)),
                                C.c_int(vec_len), _p(out))
    if rc != 0:
        raise ValueError("decode_tiles: malformed stream at vector %d" % (-rc - 1))
    return out


def fused_k(sym_tbhd, min_i8, scale_f16, mask, block_size, q):
    """F1: src/kernels.cu:293-348,721-776 in exact arithmetic.  sym u8 [T,B,H,D], q f16 [B,Hq,D] -> f64 [B,Hq,T]."""
    sym = np.ascontiguousarray(sym_tbhd, dtype=np.uint8)
    T, B, H, D = sym.shape
    q = np.ascontiguousarray(q, dtype=np.float16)
    Hq = q.shape[1]
    out = np.zeros((B, Hq, T), np.float64)
    mn = np.ascontiguousarray(min_i8, dtype=np.int8).ravel()
    sc = np.ascontiguousarray(scale_f16, dtype=np.float16).ravel()
    lib().kvo_fused_k(_p(sym), _p(mn), _p(sc.view(np.uint16)), C.c_int(mask), _i64(T), _i64(block_size), _i64(B),
                      _i64(H), _i64(D), _p(q.view(np.uint16)), _i64(Hq), _p(out))
    return out


def fused_v(sym_tbhd, min_i8, scale_f16, mask, block_size, p):
    """F2: src/kernels.cu:350-407,778-861 + kvcomp_encode.py:275.  p f16 [B,Hq,T] -> f64 [B,Hq,D]."""
    sym = np.ascontiguousarray(sym_tbhd, dtype=np.uint8)
    T, B, H, D = sym.shape
    p = np.ascontiguousarray(p, dtype=np.float16)
    Hq = p.shape[1]
    out = np.zeros((B, Hq, D), np.float64)
    mn = np.ascontiguousarray(min_i8, dtype=np.int8).ravel()
    sc = np.ascontiguousarray(scale_f16, dtype=np.float16).ravel()
    lib().kvo_fused_v(_p(sym), _p(mn), _p(sc.view(np.uint16)), C.c_int(mask), _i64(T), _i64(block_size), _i64(B),
                      _i64(H), _i64(D), _p(p.view(np.uint16)), _i64(Hq), _p(out))
    return out


def fused_k_from_stream(encoded, block_infos, thread_infos, tree, min_i8, scale_f16, q, tokens, stride, vec_len=128,
                        mask=MASK_K_BLOCK, threads=None):
    """CPU baseline: the reference's fused K kernel per lane on the host (bit-serial walk, fp16 dequant, dot).
    Returns float32 [stride/vec_len, tokens]."""
    enc = np.ascontiguousarray(encoded, dtype=np.uint8)
    tree = np.ascontiguousarray(tree, dtype=np.uint8)
    q = np.ascontiguousarray(q, dtype=np.float16)
    mn = np.ascontiguousarray(min_i8, dtype=np.int8).ravel()
    sc = np.ascontiguousarray(scale_f16, dtype=np.float16).ravel()
    out = np.zeros((stride // vec_len, tokens), np.float32)
    if threads:
        lib().kvo_set_threads(C.c_int(int(threads)))
    rc = lib().kvo_fused_k_from_stream(_p(enc), _p(np.ascontiguousarray(block_infos)),
                                       _p(np.ascontiguousarray(thread_infos)), _p(tree), _i64(tree.shape[0]),
                                       _p(mn), _p(sc.view(np.uint16)), C.c_int(mask), _p(q.view(np.uint16)), _i64(tokens),
                                       _i64(stride), C.c_int(vec_len), _p(out))
    if rc != 0:
        raise ValueError("malformed stream at vector %d" % (-rc - 1))
    return out


# ---------------------------------------------------------------------------------------------------
# Pure-Python restatements used as independent pins of the C functions above (small inputs only).
# ---------------------------------------------------------------------------------------------------
class _FreqOnly:
    """Heap item that compares on frequency only, like utils/huffman.py:13-14."""
    __slots__ = ("f", "sym", "left", "right")

    def __init__(self, f, sym=None, left=None, right=None):
        self.f, self.sym, self.left, self.right = f, sym, left, right

    def __lt__(self, other):
        return self.f < other.f


def py_huffman_codebook(symbols):
    """utils/huffman.py:15-81 through the stdlib heapq: {symbol: '0101'} for an iterable of ints."""
    vals, cnts = np.unique(np.asarray(symbols).ravel(), return_counts=True)
    if len(vals) == 0:
        return {}
    if len(vals) == 1:
        return {int(vals[0]): "0"}
    heap = []
    for s, c in zip(vals.tolist(), cnts.tolist()):
        heapq.heappush(heap, _FreqOnly(c, sym=s))
    while len(heap) > 1:
        a = heapq.heappop(heap)
        b = heapq.heappop(heap)
        heapq.heappush(heap, _FreqOnly(a.f + b.f, left=a, right=b))
    book = {}
    stack = [(heap[0], "")]
    while stack:
        node, code = stack.pop()
        if node.sym is not None:
            book[node.sym] = code or "0"
        else:
            stack.append((node.right, code + "1"))
            stack.append((node.left, code + "0"))
    return book


def py_bits(symbols, book):
    """utils/huffman.py:83-95: bool array of the concatenated code strings."""
    s = "".join(book[int(v)] for v in np.asarray(symbols).ravel().tolist())
    return np.frombuffer(s.encode(), dtype=np.uint8) == ord("1")
