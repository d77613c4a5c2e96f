"""kvc_attention_decode_static (the decode-attention entry point that allocates nothing: its workspace is a
device array inside the library) against kvc_attention_decode with a caller's workspace, through the C ABI.

Two calls in a row share the library's array, the second on a smaller cache, so whatever the first call left
in the array lies beyond (and under) what the second one uses; both must equal the existing entry point bit
for bit, since the kernels and their launch shapes are the same."""
import ctypes as C

import pytest
import torch

from tests import _synth as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _contexts(T, B, H, D, k_mode="ChannelQuant"):
    from kvcomp_amd.ctx import KVCompCacheConfig, KVCompCacheConfigStatic, KVCompCtx, QuantMode
    KVCompCacheConfigStatic.config = KVCompCacheConfig("synthetic", QuantMode(k_mode), QuantMode("TokenQuant"), 64, 128,
                                                       64, 128, 0.1, 0.2)
    k, v = S.synth_k(T, B, H, D).to(DEV), S.synth_v(T, B, H, D).to(DEV)
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k)
    vctx.store(v)
    return kctx, vctx


def _both(T, B, H, D, rep, k_mode="ChannelQuant"):
    from kvcomp_amd import _lib
    from kvcomp_amd.attention import CompressedAttention
    L = _lib.lib()
    kctx, vctx = _contexts(T, B, H, D, k_mode)
    assert kctx.ctx_len == T and vctx.ctx_len == T
    att = CompressedAttention(kctx, vctx)
    q = S.synth_q(B, H * rep, D).to(DEV).contiguous()
    scale = 1.0 / D ** 0.5
    k_lut, v_lut = att._luts()
    kd, vd = att._desc(kctx, k_lut), att._desc(vctx, v_lut)
    stream = C.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
    # the existing entry point, workspace from the caller (filled with a pattern: its contents are ignored)
    need = int(L.kvc_attention_workspace_bytes(T, vctx.compressed_ctx_len, B, H * rep, D))
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device=DEV)
    ref = torch.empty(B, H * rep, D, dtype=torch.float32, device=DEV)
    _lib.check(L.kvc_attention_decode(C.byref(kd), C.byref(vd), C.c_void_p(q.data_ptr()), scale, C.c_void_p(ws.data_ptr()),
                                      need, C.c_void_p(ref.data_ptr()), B, H, H * rep, D, None, None, stream))
    out = torch.full((B, H * rep, D), float("nan"), dtype=torch.float32, device=DEV)
    _lib.check(L.kvc_attention_decode_static(C.byref(kd), C.byref(vd), C.c_void_p(q.data_ptr()), scale,
                                             C.c_void_p(out.data_ptr()), B, H, H * rep, D, stream))
    torch.cuda.synchronize()
    return out, ref, att, q


def test_static_workspace_attention_equals_the_workspace_version_twice():
    # first call: 2048 + 40 tokens (so both fp16 tails exist), two sequences, two query heads per KV head
    out1, ref1, att1, q1 = _both(2048 + 40, 2, 4, 128, 2)
    assert torch.isfinite(ref1).all() and torch.equal(out1, ref1)
    # second call right after it, on a smaller cache of another shape (head_dim 96, one query head per KV head)
    out2, ref2, att2, q2 = _both(640, 1, 4, 96, 1, k_mode="BlockQuant")
    assert torch.isfinite(ref2).all() and torch.equal(out2, ref2)
    # and the operator is the right one: the same attention from the reference-shaped pieces, within 1e-3
    step = att2.attend_stepwise(q2)
    assert (out2 - step).abs().max() <= 1e-3 * step.abs().max()


def test_static_workspace_rejects_shapes_beyond_its_size():
    from kvcomp_amd import _lib
    L = _lib.lib()
    kd, vd = _lib.CompressedDesc(), _lib.CompressedDesc()
    kd.tokens = vd.tokens = 1 << 22                      # 4 Mi tokens x 4 x 32 heads of fp32 scores: 2 GiB
    out = torch.empty(4, 32, 128, dtype=torch.float32, device=DEV)
    q = torch.empty(4, 32, 128, dtype=torch.float16, device=DEV)
    rc = L.kvc_attention_decode_static(C.byref(kd), C.byref(vd), C.c_void_p(q.data_ptr()), 1.0, C.c_void_p(out.data_ptr()),
                                       4, 32, 32, 128, None)
    assert rc != 0 and b"static one holds" in L.kvc_last_error()
