"""Rotary position encoding with rotate-half pairing, optionally with llama3 frequency scaling.

Frequencies as the reference builds them (``base/src/kernels.cu:56-106``), in fp32:

    inv_freq_i = 1 / theta^(2i / rot),  i in [0, rot/2)
    llama3 scaling, with wavelen = 2 pi / inv_freq_i, low_wl = orig / low_freq_factor,
    high_wl = orig / high_freq_factor:
        wavelen >  low_wl            -> inv_freq_i / factor
        high_wl <= wavelen <= low_wl -> smooth = (orig / wavelen - low) / (high - low)
                                        (1 - smooth) * inv_freq_i / factor + smooth * inv_freq_i
        otherwise                    -> unchanged
    angle = position * inv_freq (fp32), tables cos(angle), sin(angle) of shape [positions, rot/2]

The tables are applied by the ``rope_kv_write`` kernel.  The frequency function is the only
thing scaling changes; another rotary variant passes other tables, another pairing needs its own
``apply_and_cache``.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from ..config.registry import POSITION_ENCODINGS
from ..ops import kernels as K
from .base import KVView, PositionEncoding


def rotary_inv_freq(rot_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    f32 = np.float32
    i = np.arange(rot_dim // 2, dtype=f32)
    inv = (f32(1.0) / np.power(f32(theta), (f32(2.0) * i) / f32(rot_dim), dtype=f32)).astype(f32)
    if not scaling:
        return inv
    factor = f32(scaling["factor"])
    low, high = f32(scaling["low_freq_factor"]), f32(scaling["high_freq_factor"])
    orig = f32(scaling["original_max_position_embeddings"])
    low_wl, high_wl = orig / low, orig / high
    out = inv.copy()
    for j in range(inv.shape[0]):
        wavelen = f32(2.0) * f32(math.pi) / inv[j]
        if wavelen > low_wl:
            out[j] = inv[j] / factor
        elif wavelen >= high_wl:
            smooth = (orig / wavelen - low) / (high - low)
            out[j] = (f32(1.0) - smooth) * (inv[j] / factor) + smooth * inv[j]
    return out.astype(f32)


# cos/sin tables shared by every encoding with the same frequencies, length and device: the
# layers of a model all rotate alike, and a table for 131,072 positions is tens of megabytes
_TABLES: "dict" = {}
_TABLES_KEPT = 8


def shared_tables(inv_freq: np.ndarray, max_positions: int, device) -> tuple:
    key = (inv_freq.tobytes(), int(max_positions), str(torch.device(device)))
    hit = _TABLES.pop(key, None)
    if hit is None:
        pos = np.arange(max_positions, dtype=np.float32)[:, None]
        angle = (pos * inv_freq[None, :]).astype(np.float32)
        hit = (torch.from_numpy(np.cos(angle).astype(np.float32)).to(device),
               torch.from_numpy(np.sin(angle).astype(np.float32)).to(device))
    _TABLES[key] = hit                      # most recently used last
    while len(_TABLES) > _TABLES_KEPT:
        _TABLES.pop(next(iter(_TABLES)))
    return hit


@POSITION_ENCODINGS.register("rotary")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, *, head_dim: int, max_positions: int, theta: float,
                 scaling: Optional[dict] = None, rotary_dim: Optional[int] = None):
        super().__init__("")
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        self.max_positions = int(max_positions)
        self.inv_freq = rotary_inv_freq(self.rotary_dim, theta, scaling)
        self._cos: Optional[torch.Tensor] = None
        self._sin: Optional[torch.Tensor] = None

    def tables(self, device) -> tuple:
        if self._cos is None or self._cos.device != torch.device(device):
            self._cos, self._sin = shared_tables(self.inv_freq, self.max_positions, device)
        return self._cos, self._sin

    def rotate_half_tables(self, device, head_dim: int):
        if self.rotary_dim != head_dim:
            return None
        return self.tables(device)

    def apply_and_cache(self, qkv, positions, num_q_heads, num_kv_heads, head_dim, kv: Optional[KVView]):
        cos, sin = self.tables(qkv.device)
        write = kv is not None and kv.writes
        K.rope_kv_write(qkv, positions, num_q_heads, num_kv_heads, head_dim, cos, sin,
                        kv.k_cache if write else None, kv.v_cache if write else None,
                        kv.slot_mapping if write else None, kv.page_size if kv is not None else 0)


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    """No encoding: Q and K pass unchanged; K and V are still written to the cache."""

    graph_safe = True

    def __init__(self, **_ignored):
        super().__init__("")

    def rotate_half_tables(self, device, head_dim: int):
        return (None, None)

    def apply_and_cache(self, qkv, positions, num_q_heads, num_kv_heads, head_dim, kv: Optional[KVView]):
        write = kv is not None and kv.writes
        if not write:
            return
        K.rope_kv_write(qkv, positions, num_q_heads, num_kv_heads, head_dim, None, None,
                        kv.k_cache, kv.v_cache, kv.slot_mapping, kv.page_size)
