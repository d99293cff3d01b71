"""Position encodings of the attention mixer.

``rotary``: rotation by pos * f_i on pairs of every query and key head
(crates/spite-rope/src/lib.rs:78-92; half-split pairs (i, i+hd/2) as there, or adjacent
pairs), f_i = theta^(-2i/hd), optionally rescaled once at load by the ``llama3`` rule
(wavelength L = 2*pi/f: L < orig/high keeps f; L > orig/low gives f/factor; between, the
blend (1-s)*f/factor + s*f with s = (orig/L - low)/(high - low)).  The table is computed in
float64 and stored as fp32; angle and rotation are fp32 in the kernel.

``none``: no position information (NoPE layers).
"""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding, register


def inv_frequencies(head_dim: int, theta: float, scaling=None):
    half = head_dim // 2
    out = []
    for i in range(half):
        f = 1.0 / (float(theta) ** (2.0 * i / head_dim))
        if scaling is not None:
            factor, low, high, orig = (float(scaling["factor"]), float(scaling["low_freq_factor"]),
                                       float(scaling["high_freq_factor"]),
                                       float(scaling["original_max_position_embeddings"]))
            wavelen = 2.0 * math.pi / f
            if wavelen < orig / high:
                pass
            elif wavelen > orig / low:
                f = f / factor
            else:
                s = (orig / wavelen - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


@register("position", "rotary")
class Rotary(PositionEncoding):
    graph_safe = True

    def __init__(self, env, head_dim: int, theta: float, scaling=None, pairing: str = "half", rotary_dim=None):
        """``rotary_dim``: only the first so many elements of a head rotate, with the frequencies of
        a head of that size; the rest pass through (default: the whole head)."""
        rot = head_dim if rotary_dim is None else int(rotary_dim)
        if head_dim % 2 or rot % 2 or not 0 < rot <= head_dim:
            raise ValueError(f"rotary: head size {head_dim} and rotating part {rot} must be even, the part within the head")
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"rotary: pairing {pairing!r}")
        if scaling is not None and scaling.get("rope_type", "llama3") != "llama3":
            raise ValueError(f"rotary: scaling of type {scaling.get('rope_type')!r} is not known")
        self.adjacent = pairing == "adjacent"
        self.rotary_dim = rot
        self.inv_freq = torch.tensor(inv_frequencies(rot, theta, scaling), dtype=torch.float64) \
            .to(torch.float32).to(env.device)

    def kernel_args(self):
        return {"use_rope": True, "inv_freq": self.inv_freq, "adjacent": self.adjacent, "rotary_dim": self.rotary_dim}


@register("position", "none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, env):
        pass
