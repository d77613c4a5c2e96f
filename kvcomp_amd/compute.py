"""Host-side mirror of the reference's utils/compute.py for the kernel path, backed by libkvcomp_hip.

Same names and argument meaning as the reference (utils/compute.py:5-143); the quantizer and dequantizer run
as HIP kernels through the C ABI, the tail bookkeeping (`cut_tensor*`, `safe_cat`) is plain tensor slicing.
"""
import ctypes as C
from enum import Enum
from typing import List, Optional, Tuple

import torch

from . import _lib
from ._lib import KvcompError, check


class QuantMode(Enum):
    """utils/compute.py:5-10"""
    BlockQuant = "BlockQuant"
    ChannelQuant = "ChannelQuant"
    TokenQuant = "TokenQuant"
    VectorQuant = "VectorQuant"


# utils/compute.py:138-143 -- reduced dimensions on the sim path's [B, H, NB, BS, D] view
QUANT_DIM = {
    QuantMode.BlockQuant.value: [1, 3, 4],
    QuantMode.ChannelQuant.value: [3],
    QuantMode.TokenQuant.value: [1, 4],
    QuantMode.VectorQuant.value: [4],
}

# models/cache/kvcomp_encode.py:10-13 -- reduced dimensions on the kernel path's [NB, BS, B, H, D] view
QUANT_MODE_MAP = {
    QuantMode.BlockQuant: [1, 2, 3, 4],
    QuantMode.TokenQuant: [2, 3, 4],
    QuantMode.ChannelQuant: [1],
    QuantMode.VectorQuant: [4],
}


def dims_to_mask(quant_dims: List[int]) -> int:
    """Reduced dimensions of a [NB, BS, B, H, D] tensor -> group mask of the C ABI (BS=1, B=2, H=4, D=8)."""
    mask = 0
    for d in quant_dims:
        d = d % 5
        if d == 0:
            raise KvcompError("the block dimension (0) cannot be reduced over")
        mask |= 1 << (d - 1)
    return mask


def mask_keepdim_shape(shape5, mask):
    NB, BS, B, H, D = shape5
    return (NB, 1 if mask & 1 else BS, 1 if mask & 2 else B, 1 if mask & 4 else H, 1 if mask & 8 else D)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream(t):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def quant(tensor: torch.Tensor, quant_dims: List[int], quant_scale_rel: float,
          counts: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """utils/compute.py:93-106 on a device fp16 [NB, BS, B, H, D] tensor.

    Returns (quant_ints - min_ints, min_ints, quant_scale) with keepdim shapes like the reference, but
    already cast the way its only caller casts them (models/cache/kvcomp_encode.py:97-98): symbols uint8,
    min_ints int8, scale fp16 -- bit-identical to the reference's fp16 op chain followed by those casts.
    `counts` (int64[256], device) optionally accumulates the symbol histogram."""
    if tensor.dim() != 5 or tensor.dtype != torch.float16 or not tensor.is_cuda:
        raise KvcompError("quant expects a device float16 tensor of shape [NB, BS, B, H, D]")
    tensor = tensor.contiguous()
    mask = dims_to_mask(quant_dims)
    gshape = mask_keepdim_shape(tensor.shape, mask)
    sym = torch.empty(tensor.shape, dtype=torch.uint8, device=tensor.device)
    min_i8 = torch.empty(gshape, dtype=torch.int8, device=tensor.device)
    scale = torch.empty(gshape, dtype=torch.float16, device=tensor.device)
    NB, BS, B, H, D = tensor.shape
    with torch.cuda.device(tensor.device):
        check(_lib.lib().kvc_quant(_ptr(tensor), NB, BS, B, H, D, mask, float(quant_scale_rel), _ptr(sym), _ptr(min_i8),
                                   _ptr(scale), None, _ptr(counts), _stream(tensor)))
    return sym, min_i8, scale


def dequant(quant_ints: torch.Tensor, min_ints: torch.Tensor, quant_scale: torch.Tensor, quant_dims: List[int]) -> torch.Tensor:
    """(decoded + min_ints) * quant_scale of models/cache/kvcomp_encode.py:146 as one kernel."""
    if quant_ints.dim() != 5 or quant_ints.dtype != torch.uint8 or not quant_ints.is_cuda:
        raise KvcompError("dequant expects a device uint8 tensor of shape [NB, BS, B, H, D]")
    quant_ints = quant_ints.contiguous()
    mask = dims_to_mask(quant_dims)
    NB, BS, B, H, D = quant_ints.shape
    out = torch.empty(quant_ints.shape, dtype=torch.float16, device=quant_ints.device)
    with torch.cuda.device(quant_ints.device):
        check(_lib.lib().kvc_dequant(_ptr(quant_ints), _ptr(min_ints.contiguous()), _ptr(quant_scale.contiguous()),
                                     NB, BS, B, H, D, mask, _ptr(out), _stream(quant_ints)))
    return out


# Simulated quantization on the sim path's [B, H, NB, BS, D] view (utils/compute.py:74-91,108-133).  The groups
# of ChannelQuant ([3]) and VectorQuant ([4]) are contiguous runs of that layout as it stands; BlockQuant
# ([1, 3, 4]) and TokenQuant ([1, 4]) reduce over the head dimension, which has to sit inside the block first.
_SIM_PLAN = {
    QuantMode.ChannelQuant: (False, 0x1),
    QuantMode.VectorQuant: (False, 0x8),
    QuantMode.TokenQuant: (True, 0xC),
    QuantMode.BlockQuant: (True, 0xD),
}


def quant_dequant_sim(tensor: torch.Tensor, block_size: int, quant_scale_rel: float, quant_mode: QuantMode) -> torch.Tensor:
    """`(quant_int + min_quant) * quant_scale` of utils/compute.py:124-131 for a device fp16 [B, H, T, D] tensor
    (T a multiple of block_size), bit-identical to the reference's chain of fp16 tensor ops, as one kernel."""
    if tensor.dim() != 4 or tensor.dtype != torch.float16 or not tensor.is_cuda:
        raise KvcompError("quant_dequant_sim expects a device float16 tensor of shape [B, H, T, D]")
    B, H, T, D = tensor.shape
    if T % block_size != 0:
        raise KvcompError("Tensor shape is not divisible by block size")
    heads_inside, mask = _SIM_PLAN[quant_mode]
    NB = T // block_size
    if heads_inside:
        x = tensor.permute(0, 2, 1, 3).contiguous()                    # [B, T, H, D]
        shape5 = (B * NB, block_size, 1, H, D)
    else:
        x = tensor.contiguous()
        shape5 = (B * H * NB, block_size, 1, 1, D)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        check(_lib.lib().kvc_quant_error(_ptr(x), *shape5, mask, float(quant_scale_rel), _ptr(out), _stream(x)))
    return out.permute(0, 2, 1, 3) if heads_inside else out


def quant_error(error_cache, buffer, new_tensor, block_size: int, recent_size: int, quant_scale_rel: float,
                quant_mode: QuantMode):
    """utils/compute.py:108-133: append to the tail, replace the whole blocks that leave it by their
    simulated-quantization values and append those to `error_cache`."""
    to_compress, in_buffer = cut_tensor(buffer, new_tensor, block_size, recent_size, dim=2)
    if to_compress is not None:
        to_compress = quant_dequant_sim(to_compress, block_size, quant_scale_rel, quant_mode)
    return safe_cat(error_cache, to_compress, dim=2), in_buffer


def safe_cat(t1, t2, dim):
    """utils/compute.py:35-42"""
    if t1 is None and t2 is None:
        return None
    if t1 is None:
        return t2.clone()
    if t2 is None:
        return t1.clone()
    return torch.cat([t1, t2], dim=dim)


def blocks_to_compress(length: int, block_size: int, recent_size: int) -> int:
    """Block count formula of utils/compute.py:51-52 / :66-67."""
    return (length + block_size - length % block_size - recent_size) // block_size


def cut_tensor_ctx_len_0(buffer, new_tensor, block_size, recent_size, dim=0):
    """utils/compute.py:59-72: append to the tail, split off the leading whole blocks that leave it."""
    buffer = safe_cat(buffer, new_tensor, dim)
    n = blocks_to_compress(buffer.shape[0], block_size, recent_size)
    to_compress = None
    if n > 0:
        to_compress = buffer[:n * block_size]
        buffer = buffer[n * block_size:]
    return to_compress, buffer


def cut_tensor(buffer, new_tensor, block_size, recent_size, dim=2):
    """utils/compute.py:44-57 (sim-path layout [B, H, T, D])."""
    buffer = safe_cat(buffer, new_tensor, dim)
    n = blocks_to_compress(buffer.shape[dim], block_size, recent_size)
    to_compress = None
    if n > 0:
        to_compress = buffer[:, :, :n * block_size, :]
        buffer = buffer[:, :, n * block_size:, :]
    return to_compress, buffer


def rotate_half(x):
    """utils/compute.py:12-16"""
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb_single(t, cos, sin, position_ids=None, unsqueeze_dim=1):
    """utils/compute.py:25-33"""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (t * cos) + (rotate_half(t) * sin)


def expected_groups(compressed_ctx_len: int, block_size: int, batch: int, heads: int, head_dim: int, quant_dims) -> int:
    """Number of (min, scale) pairs of a stream: one per combination of the dimensions of [NB, BS, B, H, D] that the
    quantizer does not reduce over (utils/compute.py:93-106)."""
    shape5 = (compressed_ctx_len // block_size, block_size, batch, heads, head_dim)
    n = 1
    for i, extent in enumerate(shape5):
        if i not in quant_dims:
            n *= extent
    return n
