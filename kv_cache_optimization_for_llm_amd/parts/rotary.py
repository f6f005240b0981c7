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


def plain_frequencies_f64(rot_dim: int, theta: float) -> np.ndarray:
    """``theta^(-2i / rot)`` in float64: tables built from these hold the correctly rounded cos and
    sin of ``position * frequency`` (an fp32 frequency times an fp32 position is off by up to
    ``position * 6e-8`` radians)."""
    i = np.arange(rot_dim // 2, dtype=np.float64)
    return np.power(np.float64(theta), -2.0 * i / np.float64(rot_dim))


def linear_frequencies_f64(rot_dim: int, theta: float, *, factor: float) -> np.ndarray:
    """Linear scaling (position interpolation): every plain frequency divided by ``factor``; float64."""
    if not factor > 0:
        raise ValueError(f"linear rotary scaling: factor {factor} must be positive")
    return plain_frequencies_f64(rot_dim, theta) / np.float64(factor)


def yarn_frequencies(rot_dim: int, theta: float, *, factor: float, original: float, fast: float,
                     slow: float) -> np.ndarray:
    """YaRN: pair i keeps its plain frequency ``f_i`` where it turns fast and takes ``f_i / factor``
    where it turns slowly, blended linearly over the pair index between the pairs that make
    ``fast`` and ``slow`` turns over ``original`` positions:
    ``index(t) = rot ln(original / (2 pi t)) / (2 ln theta)``, ``lo = max(floor(index(fast)), 0)``,
    ``hi = min(ceil(index(slow)), rot - 1)``, ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``,
    ``f_i / factor * ramp_i + f_i * (1 - ramp_i)``.  float64.  (The rotation's magnitude,
    ``0.1 ln(factor) + 1``, is the encoding's ``magnitude``: :func:`yarn_magnitude`.)"""
    f = plain_frequencies_f64(rot_dim, theta)

    def index(turns: float) -> float:
        return rot_dim * math.log(float(original) / (2.0 * math.pi * float(turns))) / (2.0 * math.log(float(theta)))

    lo = max(math.floor(index(fast)), 0)
    hi = min(math.ceil(index(slow)), rot_dim - 1)
    i = np.arange(rot_dim // 2, dtype=np.float64)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / float(factor) * ramp + f * (1.0 - ramp)


def yarn_magnitude(factor: float) -> float:
    return 0.1 * math.log(float(factor)) + 1.0


# The rule that turns (rotary width, theta, parameters) into frequencies is chosen by name; another
# scaling scheme is another entry here, registered from anywhere.
ROTARY_FREQUENCIES.register("plain", plain_frequencies, replace=True)
ROTARY_FREQUENCIES.register("llama3", llama3_frequencies, replace=True)
ROTARY_FREQUENCIES.register("plain_f64", plain_frequencies_f64, replace=True)
ROTARY_FREQUENCIES.register("yarn", yarn_frequencies, replace=True)
ROTARY_FREQUENCIES.register("linear_f64", linear_frequencies_f64, replace=True)


def rotary_inv_freq(rot_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """Frequencies for a ``rope_scaling`` dictionary as ``config.json`` holds it (``None``: plain):
    its ``rope_type`` names the rule, its other keys are the rule's parameters."""
    if not scaling:
        return plain_frequencies(rot_dim, theta)
    params = {k: v for k, v in scaling.items() if k not in ("rope_type", "type")}
    rule = scaling.get("rope_type", scaling.get("type", "plain"))
    return ROTARY_FREQUENCIES.get("plain" if rule in (None, "default") else rule)(rot_dim, theta, **params)


class _Tables:
    """cos and sin of position * frequency (times ``magnitude``), ``[positions, rot / 2]`` fp32 on
    one device.  Angles are formed in the frequencies' own type: fp32 frequencies give the fp32
    product, float64 frequencies the exact angle, rounded once at the end."""

    def __init__(self, inv_freq: np.ndarray, positions: int, device, magnitude: float = 1.0):
        kind = inv_freq.dtype.type
        pos = np.arange(positions, dtype=kind)[:, None]
        angle = (pos * inv_freq[None, :]).astype(kind)
        cos, sin = np.cos(angle), np.sin(angle)
        if magnitude != 1.0:
            cos, sin = cos * kind(magnitude), sin * kind(magnitude)
        self.cos = torch.from_numpy(cos.astype(np.float32)).to(device)
        self.sin = torch.from_numpy(sin.astype(np.float32)).to(device)


# Tables are shared by every encoding with the same frequencies, length and device (the layers of
# a model all rotate alike, and a table for 131,072 positions is tens of megabytes), and held only
# through the encodings that use them: when the last model that rotates this way is gone, so is
# its table.
_TABLES: "weakref.WeakValueDictionary" = weakref.WeakValueDictionary()


def shared_tables(inv_freq: np.ndarray, positions: int, device, magnitude: float = 1.0) -> _Tables:
    key = (inv_freq.tobytes(), str(inv_freq.dtype), float(magnitude), int(positions), str(torch.device(device)))
    hit = _TABLES.get(key)
    if hit is None:
        hit = _TABLES[key] = _Tables(inv_freq, int(positions), device, magnitude)
    return hit


@POSITION_ENCODINGS.register("rotary")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, *, head_dim: int, max_positions: int, theta: float, frequencies: str = "plain",
                 frequency_params: Optional[dict] = None, rotary_dim: Optional[int] = None,
                 pairing: str = "half", magnitude: float = 1.0, unit_norm_eps: Optional[float] = None):
        """``pairing``: pair i of the rotated elements is (i, i + rot / 2) (``"half"``) or
        (2i, 2i + 1) (``"interleaved"``).  ``magnitude`` multiplies cos and sin.  With
        ``unit_norm_eps`` every query and key head is divided by its root mean square
        (``sqrt(mean(x^2) + eps)``, over the whole head) after the rotation and before the key is
        cached."""
        super().__init__("")
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary pairing {pairing!r} is not one of 'half', 'interleaved'")
        self.pairing, self.magnitude = pairing, float(magnitude)
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        self.max_positions = int(max_positions)
        self.inv_freq = np.asarray(ROTARY_FREQUENCIES.get(frequencies)(
            self.rotary_dim, theta, **(frequency_params or {})))
        if self.inv_freq.dtype != np.float64:
            self.inv_freq = self.inv_freq.astype(np.float32)
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
            self._tables = shared_tables(self.inv_freq, self.max_positions, device, self.magnitude)
        return self._tables.cos, self._tables.sin

    def rotate_half_tables(self, device, head_dim: int):
        if self.rotary_dim != head_dim or self.pairing != "half" or self.unit_norm_eps is not None:
            return None
        return self.tables(device)

    def apply_and_cache(self, qkv, positions, num_q_heads, num_kv_heads, head_dim, kv: Optional[KVView],
                        value_dim: Optional[int] = None):
        cos, sin = self.tables(qkv.device)
        write = kv is not None and kv.writes
        value_dim = head_dim if value_dim is None else int(value_dim)
        if self.pairing != "half" or self.unit_norm_eps is not None or value_dim != head_dim:
            K.qk_encode_cache(qkv, positions, num_q_heads, num_kv_heads, head_dim, value_dim, cos, sin,
                              self.pairing == "interleaved", self.unit_norm_eps,
                              kv.k_cache if write else None, kv.v_cache if write else None,
                              kv.slot_mapping if write else None)
            return
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

    def apply_and_cache(self, qkv, positions, num_q_heads, num_kv_heads, head_dim, kv: Optional[KVView],
                        value_dim: Optional[int] = None):
        write = kv is not None and kv.writes
        if not write:
            return
        if value_dim is not None and value_dim != head_dim:
            K.qk_encode_cache(qkv, positions, num_q_heads, num_kv_heads, head_dim, value_dim, None, None, False,
                              None, kv.k_cache, kv.v_cache, kv.slot_mapping)
            return
        K.rope_kv_write(qkv, positions, num_q_heads, num_kv_heads, head_dim, None, None,
                        kv.k_cache, kv.v_cache, kv.slot_mapping, kv.page_size)
