"""ctypes front end of oracle/_ref/libkvc_ref.so: the REFERENCE's own host C++ (src/huffman.cpp,
src/compute.cpp) compiled in place by oracle/build_oracle.py.  TEST INFRASTRUCTURE ONLY.

The library is absent when the reference checkout was never mounted (it is git-ignored and only travels
as a prebuilt file); available() says whether it can be used."""
import ctypes as C
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "libkvc_ref.so")
_LIB = None


def available():
    if not os.path.exists(_PATH):
        return False
    try:
        lib()
        return True
    except OSError:
        return False


def lib():
    global _LIB
    if _LIB is None:
        import torch  # noqa: F401  (libtorch must be loaded first)
        L = C.CDLL(_PATH)
        L.kvr_cut_rows.restype = C.c_int64
        _LIB = L
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def build_codebook(symbols):
    """Reference build_codebook (src/huffman.cpp:99-157): (shift, encode_table u8, decode_tree u8)."""
    sym = np.ascontiguousarray(symbols, dtype=np.uint8).ravel()
    enc = np.zeros(256 * 8, np.uint8)
    dec = np.zeros(1024 * 3, np.uint8)
    shift = C.c_int(0)
    eb, db = C.c_int64(0), C.c_int64(0)
    rc = lib().kvr_build_codebook(_p(sym), C.c_int64(sym.shape[0]), C.byref(shift), _p(enc), C.c_int64(enc.size),
                                  C.byref(eb), _p(dec), C.c_int64(dec.size), C.byref(db))
    assert rc == 0
    return shift.value, enc[:eb.value].copy(), dec[:db.value].copy()


def quant(x, dims, eb):
    """Reference C++ quant (src/compute.cpp:40-58): (sym f16, min f16, scale f16), metadata flattened."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    shape = np.array(x.shape, np.int64)
    d = np.array(dims, np.int64)
    groups = 1
    for i, s in enumerate(x.shape):
        if i not in dims:
            groups *= s
    sym = np.empty(x.shape, np.uint16)
    mn = np.empty(groups, np.uint16)
    sc = np.empty(groups, np.uint16)
    rc = lib().kvr_quant(_p(x.view(np.uint16)), _p(shape), _p(d), C.c_int(len(dims)), C.c_float(eb), _p(sym),
                         _p(mn), C.c_int64(groups), _p(sc))
    assert rc == 0
    return sym.view(np.float16), mn.view(np.float16), sc.view(np.float16)


def cut_rows(buffer_len, new_len, block_size, recent_size):
    """Rows the reference's cut_tensor (src/compute.cpp:13-38) hands to the compressor."""
    return int(lib().kvr_cut_rows(C.c_int64(buffer_len), C.c_int64(new_len), C.c_int64(block_size),
                                  C.c_int64(recent_size)))
