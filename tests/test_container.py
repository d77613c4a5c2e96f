"""Container of a compressed stream (kvcomp_amd/container.py): framing and validation on the CPU, and on the GPU a
save -> load round trip after which decode, dequantized cache, fused attention and further appends behave
exactly as on the original context."""
import struct

import numpy as np
import pytest
import torch

from tests import _synth as S


class _Stub:
    """The attributes dumps() reads, with CPU tensors (no kernel involved)."""
    is_k = True
    batch_size, head_num, head_dim = 1, 2, 8
    quant_scale_rel, quant_dims, block_size, recent_size = 0.1, [1], 64, 64
    ctx_len, compressed_ctx_len, max_code_bits, max_tile_bytes, max_stream_bytes = 70, 64, 5, 100, 9
    tree_format = 3
    encode_codebook = torch.arange(16, dtype=torch.uint8)
    decode_codebook = torch.arange(6, dtype=torch.uint8)
    block_infos = torch.zeros(16, dtype=torch.uint8)
    thread_infos = torch.ones(256, dtype=torch.uint8)
    quant_min_ints = torch.zeros(1, 1, 1, 2, 8, dtype=torch.int8)
    quant_scales = torch.ones(1, 1, 1, 2, 8, dtype=torch.float16)
    encoded_data = torch.arange(100, dtype=torch.uint8)
    buffer = torch.ones(6, 1, 2, 8, dtype=torch.float16)


def test_framing_alignment_and_validation():
    from kvcomp_amd import container as Cn
    blob = Cn.dumps(_Stub())
    assert blob[:8] == Cn.MAGIC
    h = Cn.parse_header(blob)
    names = [s["name"] for s in h["sections"]]
    assert names == ["encode_codebook", "decode_codebook", "block_infos", "thread_infos", "quant_min_ints", "quant_scales",
                     "encoded_data", "tail"]
    for s in h["sections"]:
        assert s["offset"] % 64 == 0 and s["offset"] + s["nbytes"] <= len(blob)
    enc = next(s for s in h["sections"] if s["name"] == "encoded_data")
    assert np.array_equal(np.frombuffer(blob, np.uint8, enc["nbytes"], enc["offset"]), np.arange(100, dtype=np.uint8))
    assert h["compressed_ctx_len"] == 64 and h["quant_dims"] == [1]
    for bad in (blob[:100], b"NOTKVCMP" + blob[8:], blob[:8] + struct.pack("<Q", 1 << 40) + blob[16:], blob[:-200]):
        with pytest.raises(Cn.ContainerError):
            Cn.parse_header(bad)


def _rewrite_header(blob, edit):
    """The same container with its JSON header edited (the sections keep their places)."""
    import json
    (hlen,) = struct.unpack("<Q", blob[8:16])
    header = json.loads(blob[16:16 + hlen].decode())
    edit(header)
    body = json.dumps(header).encode()
    assert len(body) <= hlen
    return blob[:16] + body + b" " * (hlen - len(body)) + blob[16 + hlen:]


def test_inconsistent_sections_are_refused():
    """The kernels take the arrays of a stream by pointer, so a container whose sections do not fit its header's
    geometry (too few quantization parameters, a short tail, metadata of another tile count, a wrong dtype, a token
    count that is not whole tiles) must be refused before any tensor reaches the device."""
    from kvcomp_amd import container as Cn
    blob = Cn.dumps(_Stub())
    Cn.parse_header(blob)                                            # the undamaged container is fine

    def section(h, name):
        return next(s for s in h["sections"] if s["name"] == name)

    def shrink(name, shape, itemsize):
        def edit(h):
            s = section(h, name)
            s["shape"], s["nbytes"] = shape, int(np.prod(shape)) * itemsize
        return edit

    damaged = {
        "too few scales": shrink("quant_scales", [1, 1, 1, 2, 4], 2),
        "too few minima": shrink("quant_min_ints", [1, 1, 1, 1, 8], 1),
        "short tail": shrink("tail", [5, 1, 2, 8], 2),
        "tail of another head count": shrink("tail", [6, 1, 1, 8], 2),
        "block_infos of one tile only": shrink("block_infos", [8], 1),
        "thread_infos too short": shrink("thread_infos", [128], 1),
        "scales stored as bytes": lambda h: section(h, "quant_scales").update(dtype="u8", nbytes=16),
        "compressed part is not whole tiles": lambda h: h.update(compressed_ctx_len=60, ctx_len=66),
        "more compressed than stored": lambda h: h.update(ctx_len=32),
        "more heads than the sections cover": lambda h: h.update(head_num=4),
        "head_dim the kernels do not take": lambda h: h.update(head_dim=12),
        "section missing": lambda h: h["sections"].pop(3),
        "no payload": lambda h: section(h, "encoded_data").update(nbytes=0, offset=0, shape=None),
    }
    for what, edit in damaged.items():
        with pytest.raises(Cn.ContainerError):
            Cn.parse_header(_rewrite_header(blob, edit))
            pytest.fail("accepted: " + what)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [128, 96])
def test_save_load_round_trip_on_gpu(tmp_path, D):
    from kvcomp_amd import container as Cn
    from kvcomp_amd.attention import CompressedAttention
    from kvcomp_amd.ctx import KVCompCtx
    from tests.test_gpu_ctx import _config
    _config(k_mode="ChannelQuant", v_mode="TokenQuant")
    T, B, H = 512 + 37, 2, 4
    k, v = S.synth_k(T + 200, B, H, D).cuda(), S.synth_v(T + 200, B, H, D).cuda()
    kctx, vctx = KVCompCtx(True, B, H, D, 0.1), KVCompCtx(False, B, H, D, 0.2)
    kctx.store(k[:T].contiguous())
    vctx.store(v[:T].contiguous())
    Cn.save(kctx, str(tmp_path / "k.kvc"))
    Cn.save(vctx, str(tmp_path / "v.kvc"))
    k2, v2 = Cn.load(str(tmp_path / "k.kvc")), Cn.load(str(tmp_path / "v.kvc"))
    for a, b in ((kctx, k2), (vctx, v2)):
        assert (a.ctx_len, a.compressed_ctx_len, a.max_code_bits) == (b.ctx_len, b.compressed_ctx_len, b.max_code_bits)
        for name in ("encoded_data", "block_infos", "thread_infos", "quant_min_ints", "quant_scales", "buffer",
                     "encode_codebook", "decode_codebook"):
            assert torch.equal(getattr(a, name), getattr(b, name)), name
        assert torch.equal(a.get()[0], b.get()[0])
    q = S.synth_q(B, H, D).cuda()
    assert torch.equal(CompressedAttention(kctx, vctx).attend(q), CompressedAttention(k2, v2).attend(q))
    # both keep growing identically
    for i in range(T, T + 200):
        for a, b, x in ((kctx, k2, k), (vctx, v2, v)):
            a.store(x[i:i + 1].contiguous(), want_symbols=False)
            b.store(x[i:i + 1].contiguous(), want_symbols=False)
    assert kctx.compressed_ctx_len == k2.compressed_ctx_len > 512
    assert torch.equal(kctx.encoded_data, k2.encoded_data) and torch.equal(vctx.encoded_data, v2.encoded_data)
    assert torch.equal(kctx.get()[0], k2.get()[0]) and torch.equal(vctx.get()[0], v2.get()[0])
