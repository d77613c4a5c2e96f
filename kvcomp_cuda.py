"""`import kvcomp_cuda` -- the module name the reference's Python callers import
(kvcomp_cuda_extension/setup.py:18-21, models/cache/kvcomp_encode.py:6, accuracy/reproduce_cuda_error.py:2).

With this directory on sys.path the name resolves to the HIP implementation: the four constants and nine functions
of kvcomp_cuda_extension/kvcomp_cuda.pyi, same names, argument order and return values, bound to libkvcomp_hip.so
through its C ABI (kvcomp_amd/kvcomp_cuda.py).  Nothing here falls back to a CPU path: the first call raises if the
library has not been built."""
from kvcomp_amd.kvcomp_cuda import *                      # noqa: F401,F403
from kvcomp_amd.kvcomp_cuda import (K_VEC_LEN, K_VEC_PER_BLK, V_VEC_LEN, V_VEC_PER_BLK,      # noqa: F401
                                    build_codebook, calculate_buffer_size, k_decode_and_mat_vec_mul_cuda_export,
                                    k_entropy_decode_cuda_export, k_entropy_encode_cuda_export, k_mat_vec_mul_cuda_export,
                                    v_decode_and_mat_vec_mul_cuda_export, v_entropy_decode_cuda_export,
                                    v_entropy_encode_cuda_export)
