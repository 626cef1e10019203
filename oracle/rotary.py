"""CPU restatement of the reference's rotary position embedding.  Test infrastructure only:
imported by tests/ and the smoke check, never by the product path.

Follows diffulex/layer/rotary_embedding.py: the angle table of ``RotaryEmbedding.__init__``
(l.29-37) and ``apply_rotary_emb`` (l.7-17) as called by ``forward`` (l.39-66).  Pinned in
tests/test_oracle_rotary.py against an independent complex-number evaluation in float64, the
identity at position 0, norm preservation, additivity of positions and a scalar loop.
"""
from __future__ import annotations

import numpy as np
import torch


def cos_sin_cache(head_size: int, max_position: int, base: float) -> torch.Tensor:
    """[max_position, head_size] fp32: cos(t * inv_freq) then sin(t * inv_freq)  (l.29-37)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_size, 2, dtype=torch.float) / head_size))
    t = torch.arange(max_position, dtype=torch.float)
    freqs = t[:, None] * inv_freq[None, :]
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def _bf16_to_f32(x: torch.Tensor) -> np.ndarray:
    bits = x.contiguous().view(torch.int16).numpy().astype(np.uint16).astype(np.uint32) << np.uint32(16)
    return bits.view(np.float32)


def _f32_to_bf16(y: np.ndarray) -> torch.Tensor:
    """Round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(y, dtype=np.float32).view(np.uint32)
    r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    return torch.from_numpy(r.view(np.int16).copy()).view(torch.bfloat16)


def apply_rotary(x: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, head_size: int) -> torch.Tensor:
    """x: [T, H * hd] or [T, H, hd] bf16 (CPU).  Returns the rotated tensor, same shape, bf16.

    l.7-17: halves x1, x2 of every head; y1 = x1*cos - x2*sin, y2 = x2*cos + x1*sin in fp32,
    each product and the sum/difference a separately rounded operation; cast back to bf16.
    """
    shape = x.shape
    T = shape[0]
    xf = _bf16_to_f32(x).reshape(T, -1, head_size)
    cs = table[positions.long()].numpy().astype(np.float32)  # [T, hd]
    half = head_size // 2
    cos = cs[:, None, :half]
    sin = cs[:, None, half:]
    x1, x2 = xf[..., :half], xf[..., half:]
    a = (x1 * cos).astype(np.float32)
    b = (x2 * sin).astype(np.float32)
    d = (x2 * cos).astype(np.float32)
    e = (x1 * sin).astype(np.float32)
    y = np.concatenate(((a - b).astype(np.float32), (d + e).astype(np.float32)), axis=-1)
    return _f32_to_bf16(y).reshape(shape)
