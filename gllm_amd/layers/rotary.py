"""Rotary position embedding with host-precomputed cos/sin cache.

MI355X note: on-device sinf/cosf per element turns a memory-bound op
VALU-bound (cdna_hip_programming.md App. B) — the cache is built once on
host, stored [max_pos, rot_dim] as [cos | sin] halves, and the HIP
kernel just gathers it.

Scaling variants at parity with the reference
(layers/rotary_embedding.py): linear, llama3, yarn.
"""

import math
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from gllm_amd import ops


class RotaryEmbedding(nn.Module):
    def __init__(self, head_dim: int, rot_dim: int, max_position: int,
                 base: float, is_neox: bool = True,
                 scaling_factor: float = 1.0):
        super().__init__()
        self.head_dim = head_dim
        self.rot_dim = rot_dim
        self.max_position = max_position
        self.base = base
        self.is_neox = is_neox
        self.scaling_factor = scaling_factor
        cache = self._build_cache()
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def _inv_freq(self) -> torch.Tensor:
        return 1.0 / (self.base ** (
            torch.arange(0, self.rot_dim, 2, dtype=torch.float32)
            / self.rot_dim))

    def _positions(self) -> torch.Tensor:
        n = int(self.max_position * max(1.0, self.scaling_factor))
        t = torch.arange(n, dtype=torch.float32)
        if self.scaling_factor != 1.0:
            t = t / self.scaling_factor
        return t

    def _build_cache(self) -> torch.Tensor:
        inv_freq = self._inv_freq()
        t = self._positions()
        freqs = torch.outer(t, inv_freq)              # [P, rot/2]
        return torch.cat([freqs.cos(), freqs.sin()], dim=-1)  # [P, rot_dim]

    def forward(self, positions: torch.Tensor, q: torch.Tensor,
                k: torch.Tensor):
        return ops.rotary_embedding(
            positions, q, k, self.head_dim,
            self.cos_sin_cache.to(device=q.device), self.is_neox)


class Llama3RotaryEmbedding(RotaryEmbedding):
    def __init__(self, head_dim, rot_dim, max_position, base, is_neox,
                 factor, low_freq_factor, high_freq_factor,
                 original_max_position):
        self.factor = factor
        self.low_freq_factor = low_freq_factor
        self.high_freq_factor = high_freq_factor
        self.original_max_position = original_max_position
        super().__init__(head_dim, rot_dim, max_position, base, is_neox)

    def _inv_freq(self):
        inv = super()._inv_freq()
        low_wl = self.original_max_position / self.low_freq_factor
        high_wl = self.original_max_position / self.high_freq_factor
        wl = 2 * math.pi / inv
        smooth = ((self.original_max_position / wl - self.low_freq_factor)
                  / (self.high_freq_factor - self.low_freq_factor))
        smooth = smooth.clamp(0.0, 1.0)
        scaled = inv / self.factor
        blended = (1 - smooth) * scaled + smooth * inv
        out = torch.where(wl > low_wl, scaled, inv)
        mid = (wl <= low_wl) & (wl >= high_wl)
        out = torch.where(mid, blended, out)
        return out


class YaRNRotaryEmbedding(RotaryEmbedding):
    def __init__(self, head_dim, rot_dim, max_position, base, is_neox,
                 factor, original_max_position, beta_fast=32, beta_slow=1,
                 attn_factor=1.0, mscale: Optional[float] = None,
                 mscale_all_dim: Optional[float] = None):
        self.factor = factor
        self.original_max_position = original_max_position
        self.beta_fast = beta_fast
        self.beta_slow = beta_slow
        self.attn_factor = attn_factor
        if mscale is not None and mscale_all_dim is not None:
            def _ms(s, m):
                return 1.0 if s <= 1 else 0.1 * m * math.log(s) + 1.0
            self.mscale = (_ms(factor, mscale)
                           / _ms(factor, mscale_all_dim) * attn_factor)
        else:
            self.mscale = (0.1 * math.log(factor) + 1.0
                           if factor > 1 else 1.0) * attn_factor
        super().__init__(head_dim, rot_dim, max_position, base, is_neox)

    def _yarn_find_dim(self, num_rot):
        return (self.rot_dim * math.log(
            self.original_max_position / (num_rot * 2 * math.pi))
            / (2 * math.log(self.base)))

    def _inv_freq(self):
        pos_freqs = self.base ** (
            torch.arange(0, self.rot_dim, 2, dtype=torch.float32)
            / self.rot_dim)
        inv_extrap = 1.0 / pos_freqs
        inv_interp = 1.0 / (self.factor * pos_freqs)
        low = max(math.floor(self._yarn_find_dim(self.beta_fast)), 0)
        high = min(math.ceil(self._yarn_find_dim(self.beta_slow)),
                   self.rot_dim - 1)
        if low == high:
            high += 0.001
        ramp = ((torch.arange(self.rot_dim // 2, dtype=torch.float32) - low)
                / (high - low)).clamp(0, 1)
        mask = 1.0 - ramp
        return inv_interp * (1 - mask) + inv_extrap * mask

    def _positions(self):
        n = int(self.max_position * self.factor)
        return torch.arange(n, dtype=torch.float32)

    def _build_cache(self):
        inv_freq = self._inv_freq()
        t = self._positions()
        freqs = torch.outer(t, inv_freq)
        return torch.cat([freqs.cos() * self.mscale,
                          freqs.sin() * self.mscale], dim=-1)


_ROPE_CACHE: Dict[Tuple, RotaryEmbedding] = {}


def get_rope(head_dim: int, rot_dim: int, max_position: int, base: float,
             is_neox: bool = True, rope_scaling: Optional[dict] = None
             ) -> RotaryEmbedding:
    def _freeze(v):
        return tuple(v) if isinstance(v, list) else v
    key = (head_dim, rot_dim, max_position, base, is_neox,
           tuple(sorted((k, _freeze(v)) for k, v in rope_scaling.items()))
           if rope_scaling else None)
    if key in _ROPE_CACHE:
        return _ROPE_CACHE[key]
    if rope_scaling is None:
        rope = RotaryEmbedding(head_dim, rot_dim, max_position, base, is_neox)
    else:
        rtype = rope_scaling.get("rope_type",
                                 rope_scaling.get("type", "linear"))
        if rtype == "linear":
            rope = RotaryEmbedding(
                head_dim, rot_dim, max_position, base, is_neox,
                scaling_factor=rope_scaling["factor"])
        elif rtype == "llama3":
            rope = Llama3RotaryEmbedding(
                head_dim, rot_dim, max_position, base, is_neox,
                rope_scaling["factor"],
                rope_scaling.get("low_freq_factor", 1.0),
                rope_scaling.get("high_freq_factor", 4.0),
                rope_scaling.get("original_max_position_embeddings", 8192))
        elif rtype == "yarn":
            rope = YaRNRotaryEmbedding(
                head_dim, rot_dim,
                rope_scaling.get("original_max_position_embeddings",
                                 max_position),
                base, is_neox, rope_scaling["factor"],
                rope_scaling.get("original_max_position_embeddings",
                                 max_position),
                beta_fast=rope_scaling.get("beta_fast", 32),
                beta_slow=rope_scaling.get("beta_slow", 1),
                attn_factor=rope_scaling.get("attention_factor", 1.0) or 1.0,
                mscale=rope_scaling.get("mscale"),
                mscale_all_dim=rope_scaling.get("mscale_all_dim"))
        elif rtype in ("mrope", "default") and \
                rope_scaling.get("mrope_section"):
            from gllm_amd.layers.mrope import MRotaryEmbedding
            rope = MRotaryEmbedding(
                head_dim, rot_dim, max_position, base,
                list(rope_scaling["mrope_section"]),
                mrope_interleaved=bool(
                    rope_scaling.get("mrope_interleaved", False)))
        elif rtype == "default":
            rope = RotaryEmbedding(head_dim, rot_dim, max_position, base,
                                   is_neox)
        else:
            raise ValueError(f"unsupported rope_type {rtype}")
    _ROPE_CACHE[key] = rope
    return rope


class PairRotary(nn.Module):
    """Interleaved-pair rotary table: dimension 2i rotates with 2i+1 on
    the first ``rot_dims`` dims of a head, the rest pass through.

    Holds only the per-pair frequencies (fp64) and the cos/sin
    magnitude; angles are formed inside the fused q/k kernel
    (ops.qk_norm_rope_store) as position * frequency in fp64, so there is
    no max-position table to size. ``scaling`` = dict(factor, original,
    fast, slow) applies YaRN: pairs whose wavelength exceeds the original
    context (ramp 1) are slowed by ``factor``, short-wavelength pairs
    (ramp 0) keep their frequency, with a linear ramp between the
    correction dims of ``fast`` and ``slow`` rotations, and cos/sin are
    scaled by 0.1 ln(factor) + 1.

    ``scaling`` = dict(factor, low, high, original) instead selects the
    wavelength rule: with l = 2 pi / f, pairs with l < original/high
    keep f, pairs with l > original/low run at f / factor, and between
    the two f is blended linearly in s = (original/l - low) /
    (high - low): (1 - s) f / factor + s f. cos/sin keep magnitude 1.
    """

    def __init__(self, rot_dims: int, base: float,
                 scaling: Optional[dict] = None):
        super().__init__()
        assert rot_dims % 2 == 0
        self.rot_dims = rot_dims
        i = torch.arange(rot_dims // 2, dtype=torch.float64)
        freqs = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                          -2.0 * i / max(rot_dims, 1))
        self.mag = 1.0
        if scaling and "low" in scaling:
            factor = float(scaling["factor"])
            low, high = float(scaling["low"]), float(scaling["high"])
            orig = float(scaling["original"])
            wl = 2 * math.pi / freqs
            s = (orig / wl - low) / (high - low)
            blend = (1.0 - s) * freqs / factor + s * freqs
            freqs = torch.where(wl < orig / high, freqs,
                                torch.where(wl > orig / low,
                                            freqs / factor, blend))
        elif scaling:
            factor = float(scaling["factor"])
            orig = float(scaling["original"])

            def correction_dim(turns: float) -> float:
                return rot_dims * math.log(orig / (2 * math.pi * turns)) \
                    / (2 * math.log(base))

            lo = max(math.floor(correction_dim(float(scaling["fast"]))), 0)
            hi = min(math.ceil(correction_dim(float(scaling["slow"]))),
                     rot_dims - 1)
            ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
            freqs = freqs / factor * ramp + freqs * (1.0 - ramp)
            self.mag = 0.1 * math.log(factor) + 1.0
        self.register_buffer("freqs", freqs, persistent=False)


class HalfRotary(nn.Module):
    """Rotate-half rotary on the first ``rot_dims`` dims of a head:
    dimension i pairs with i + rot_dims/2 (i < rot_dims/2), frequency
    base^(-2i/rot_dims); the remaining dims pass through.

    Like PairRotary it holds only the fp64 per-pair frequencies; the
    fused q/k kernel (ops.qk_norm_rope_store with ``half_layout``) forms
    position * frequency in fp64, so no position table is sized.

    ``scaling`` = dict(factor): linear position scaling, every
    frequency divided by ``factor``.
    """

    half_layout = True
    mag = 1.0

    def __init__(self, rot_dims: int, base: float,
                 scaling: Optional[dict] = None):
        super().__init__()
        assert rot_dims % 2 == 0
        self.rot_dims = rot_dims
        i = torch.arange(rot_dims // 2, dtype=torch.float64)
        freqs = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                          -2.0 * i / max(rot_dims, 1))
        if scaling:
            extra = set(scaling) - {"factor"}
            if extra:
                raise ValueError(f"unknown rotary scaling keys {extra}")
            freqs = freqs / float(scaling.get("factor", 1.0))
        self.register_buffer("freqs", freqs, persistent=False)
