"""RMSNorm (crates/spite-models/src/dense.rs:175-181): y = x * 1/sqrt(mean(x^2) + eps) * w,
sum and scale in fp32, fused with the residual additions that precede it."""
from __future__ import annotations

import torch

from .base import Norm, ParamSpec, register
from ..csrc import hipops


@register("norm", "rms")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, env, width: int, eps: float):
        self.width = int(width)
        self.eps = float(eps)
        self.weight = None

    def params(self):
        return {"weight": ParamSpec((self.width,), kind="vector", init="ones")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def can_project(self, proj) -> bool:
        # the kernel keeps the normed row in LDS for the products
        return proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[1] == self.width \
            and hipops.add_rmsnorm_can_project(self.width)

    def forward(self, h, out, *, d1=None, d2=None, out32=None, rows=None, write_h=True, proj=None, proj_out=None):
        hipops.add_rmsnorm(h, self.weight, self.eps, out=out, out32=out32, d1=d1, d2=d2, rows=rows,
                           n_rows=(rows.numel() if rows is not None else h.shape[0]), write_h=write_h,
                           proj=proj, proj_out=proj_out)
