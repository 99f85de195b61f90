"""1-bit and 4-bit packing of byte tensors on the GPU.

Python surface of the reference's monet/lm_ops/pack.py:9-54 over the
mn_pack_* / mn_unpack_* entry points.  Formats: `pack` puts element i into
byte i//8, bit 7-(i%8); `pack_two` puts element 2j into the high nibble of
byte j.  All functions take and return 1-D contiguous GPU tensors.
"""
import torch

from .. import _lib


def _check_1d(t, name, dtype):
    _lib.require_gpu_tensor(t, name, dtype)
    if t.dim() != 1:
        raise RuntimeError("Only 1D tensors supported.")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def pack(v: torch.Tensor) -> torch.Tensor:
    """8 bools -> 1 uint8 (MSB first); output has (n+7)//8 bytes."""
    _check_1d(v, "v", torch.bool)
    n = v.numel()
    out = torch.empty((n + 7) // 8, dtype=torch.uint8, device=v.device)
    _lib.call("mn_pack_bits", _lib.ptr(v), _lib.ptr(out), n, _lib.stream_ptr(v.device))
    return out


def pack_(v: torch.Tensor, p: torch.Tensor) -> None:
    """`pack` into a caller-provided uint8 tensor of (n+7)//8 bytes."""
    _check_1d(v, "v", torch.bool)
    _check_1d(p, "p", torch.uint8)
    n = v.numel()
    if p.numel() != (n + 7) // 8:
        raise RuntimeError("Only tensors size mismatch.")
    _lib.call("mn_pack_bits", _lib.ptr(v), _lib.ptr(p), n, _lib.stream_ptr(v.device))


def unpack(p: torch.Tensor, n: int = 0) -> torch.Tensor:
    """uint8 -> 8 bools; `n` is the output length (default 8 * len(p))."""
    _check_1d(p, "p", torch.uint8)
    n = n or p.numel() * 8
    if n > p.numel() * 8:
        raise RuntimeError("n exceeds the number of packed bits")
    out = torch.empty(n, dtype=torch.bool, device=p.device)
    _lib.call("mn_unpack_bits", _lib.ptr(p), _lib.ptr(out), n, _lib.stream_ptr(p.device))
    return out


def unpack_multiply(p: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """r[i] = bit(i) * v[i] in one pass (fp32 `v`)."""
    _check_1d(p, "p", torch.uint8)
    _check_1d(v, "v", torch.float32)
    if v.device != p.device:
        raise RuntimeError("All input need to be located on the same device.")
    n = v.numel()
    if n > p.numel() * 8:
        raise RuntimeError("v is longer than the number of packed bits")
    out = torch.empty_like(v)
    _lib.call("mn_unpack_bits_mul_f32", _lib.ptr(p), _lib.ptr(v), _lib.ptr(out), n,
              _lib.stream_ptr(v.device))
    return out


def pack_two(v: torch.Tensor) -> torch.Tensor:
    """2 uint8 values (< 16) -> 1 uint8; output has (n+1)//2 bytes."""
    _check_1d(v, "v", torch.uint8)
    n = v.numel()
    out = torch.empty((n + 1) // 2, dtype=torch.uint8, device=v.device)
    _lib.call("mn_pack_nibbles", _lib.ptr(v), _lib.ptr(out), n, _lib.stream_ptr(v.device))
    return out


def unpack_two(p: torch.Tensor, n: int = 0) -> torch.Tensor:
    """uint8 -> 2 uint8 values < 16; `n` is the output length (default 2 * len(p))."""
    _check_1d(p, "p", torch.uint8)
    n = n or p.numel() * 2
    if n > p.numel() * 2:
        raise RuntimeError("n exceeds the number of packed nibbles")
    out = torch.empty(n, dtype=torch.uint8, device=p.device)
    _lib.call("mn_unpack_nibbles", _lib.ptr(p), _lib.ptr(out), n, _lib.stream_ptr(p.device))
    return out
