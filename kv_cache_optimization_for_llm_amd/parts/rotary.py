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

The tables are applied by the ``rope_kv_write`` kernel.  The frequency rule is the only thing
scaling changes, and it is a parameter of the part, chosen by name (``frequencies="llama3"`` with
its constants in ``frequency_params``; ``"plain"`` takes none): another scheme is registered in
``ROTARY_FREQUENCIES``, another pairing needs its own ``apply_and_cache``.
"""
from __future__ import annotations

import math
import weakref
from typing import Optional

import numpy as np
import torch

from ..config.registry import POSITION_ENCODINGS, ROTARY_FREQUENCIES
from ..ops import kernels as K
from .base import KVView, PositionEncoding


def plain_frequencies(rot_dim: int, theta: float) -> np.ndarray:
    f32 = np.float32
    i = np.arange(rot_dim // 2, dtype=f32)
    return (f32(1.0) / np.power(f32(theta), (f32(2.0) * i) / f32(rot_dim), dtype=f32)).astype(f32)


def llama3_frequencies(rot_dim: int, theta: float, *, factor: float, low_freq_factor: float,
                       high_freq_factor: float, original_max_position_embeddings: int) -> np.ndarray:
    f32 = np.float32
    inv = plain_frequencies(rot_dim, theta)
    factor = f32(factor)
    low, high = f32(low_freq_factor), f32(high_freq_factor)
    orig = f32(original_max_position_embeddings)
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


# The rule that turns (rotary width, theta, parameters) into frequencies is chosen by name; another
# scaling scheme is another entry here, registered from anywhere.
ROTARY_FREQUENCIES.register("plain", plain_frequencies, replace=True)
ROTARY_FREQUENCIES.register("llama3", llama3_frequencies, replace=True)


def rotary_inv_freq(rot_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """Frequencies for a ``rope_scaling`` dictionary as ``config.json`` holds it (``None``: plain):
    its ``rope_type`` names the rule, its other keys are the rule's parameters."""
    if not scaling:
        return plain_frequencies(rot_dim, theta)
    params = {k: v for k, v in scaling.items() if k not in ("rope_type", "type")}
    rule = scaling.get("rope_type", scaling.get("type", "plain"))
    return ROTARY_FREQUENCIES.get("plain" if rule in (None, "default") else rule)(rot_dim, theta, **params)


class _Tables:
    """cos and sin of position * frequency, ``[positions, rot / 2]`` fp32 on one device."""

    def __init__(self, inv_freq: np.ndarray, positions: int, device):
        pos = np.arange(positions, dtype=np.float32)[:, None]
        angle = (pos * inv_freq[None, :]).astype(np.float32)
        self.cos = torch.from_numpy(np.cos(angle).astype(np.float32)).to(device)
        self.sin = torch.from_numpy(np.sin(angle).astype(np.float32)).to(device)


# Tables are shared by every encoding with the same frequencies, length and device (the layers of
# a model all rotate alike, and a table for 131,072 positions is tens of megabytes), and held only
# through the encodings that use them: when the last model that rotates this way is gone, so is
# its table.
_TABLES: "weakref.WeakValueDictionary" = weakref.WeakValueDictionary()


def shared_tables(inv_freq: np.ndarray, positions: int, device) -> _Tables:
    key = (inv_freq.tobytes(), int(positions), str(torch.device(device)))
    hit = _TABLES.get(key)
    if hit is None:
        hit = _TABLES[key] = _Tables(inv_freq, int(positions), device)
    return hit


@POSITION_ENCODINGS.register("rotary")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, *, head_dim: int, max_positions: int, theta: float, frequencies: str = "plain",
                 frequency_params: Optional[dict] = None, rotary_dim: Optional[int] = None):
        super().__init__("")
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        self.max_positions = int(max_positions)
        self.inv_freq = np.asarray(ROTARY_FREQUENCIES.get(frequencies)(
            self.rotary_dim, theta, **(frequency_params or {})), dtype=np.float32)
        if self.inv_freq.shape != (self.rotary_dim // 2,):
            raise ValueError(f"frequency rule {frequencies!r} gave {self.inv_freq.shape[0]} frequencies for a "
                             f"rotation over {self.rotary_dim} elements")
        self._tables: Optional[_Tables] = None

    def limit_positions(self, positions: int) -> None:
        """No position at or past ``positions`` will be asked for (an engine whose longest request
        is shorter than the model's ``max_position_embeddings``): tables are built that long."""
        positions = max(1, min(int(positions), self.max_positions))
        if positions != self.max_positions:
            self.max_positions, self._tables = positions, None

    def tables(self, device) -> tuple:
        if self._tables is None or self._tables.cos.device != torch.device(device):
            self._tables = shared_tables(self.inv_freq, self.max_positions, device)
        return self._tables.cos, self._tables.sin

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
