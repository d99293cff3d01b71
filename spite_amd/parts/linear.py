"""Matrix products of the parts: picks the kernel for the dtypes and shapes at hand.

``Y = X . W^T`` with W ``[out, in]``; the grouped form walks a row list (see
``gemm_generic.hip``).  A weight that stayed in 32-bit inside a bfloat16 run is multiplied in
32-bit: the activations are widened for that product.
"""
from __future__ import annotations

import math
from typing import List

import torch

from ..csrc import hipops


def _scratch(ws, shape, dtype, device):
    """From the step's workspace when the caller has one (a warmed-up engine then allocates
    nothing inside a step), else a fresh tensor."""
    return ws.take(tuple(shape), dtype) if ws is not None else torch.empty(tuple(shape), dtype=dtype, device=device)


def _widen(x, ws=None):
    y = _scratch(ws, x.shape, torch.float32, x.device)
    hipops.convert(x, y)
    return y


SKINNY_MAX_ROWS = 64


class Weight:
    """A weight as the product kernels want it.  bfloat16 matrices whose rows are a multiple of
    16 and whose columns a multiple of 64 are kept in MFMA operand order (``hipops.operand_order``:
    a wave's operand load is then one run of whole cache lines, which the prefill products are
    bound by); everything else stays row-major.  ``shape`` is the logical ``[..., out, in]``."""

    __slots__ = ("data", "tiled", "shape", "dtype")

    def __init__(self, w: torch.Tensor, allow_tiled: bool = True):
        w = w.contiguous()
        self.shape, self.dtype = tuple(w.shape), w.dtype
        self.tiled = bool(allow_tiled and w.dtype == torch.bfloat16 and w.dim() >= 2 and w.is_cuda
                          and w.shape[-2] % 16 == 0 and w.shape[-1] % 64 == 0)
        self.data = hipops.operand_order(w) if self.tiled else w

    def slow_reason(self, name: str) -> List[str]:
        """Why products with this weight will not run on the matrix units in a bfloat16 run."""
        if self.dtype == torch.bfloat16 and self.shape[-1] % 8:
            return [f"{name} {self.shape}: rows of {self.shape[-1]} are no multiple of 8, its products run on plain FMAs"]
        if self.dtype == torch.float32:
            return [f"{name} {self.shape}: kept in 32-bit by the checkpoint, its products run on plain FMAs"]
        return []

    def group(self, g: int) -> "Weight":
        """Group ``g`` of a stack of matrices ``[groups, out, in]`` as a weight of its own (the same
        memory)."""
        one = object.__new__(Weight)
        one.data, one.tiled, one.shape, one.dtype = self.data[g], self.tiled, self.shape[1:], self.dtype
        return one


# what a tile of 160 rows costs against one of 128 (a tile's time is a fixed part and a part per
# 16 rows, 38 and 8.5 us at K = 5,120 on an MI355X: (38 + 85) / (38 + 68))
TILE_160_COST = 1.16


def grouped_tile_shape(tokens: int, groups: int, whole_groups: int = 0, col_tiles: int = 0, cus: int = 0) -> int:
    """Which tile of the prefill product suits ``tokens`` rows that spread evenly over ``groups``
    groups (experts that a router picks), beside ``whole_groups`` groups that take every row.
    A group costs whole row tiles, each of which streams the group's weights once.

    * Few rows a group and few groups (a short prompt over a few experts): the time is the stream
      of the weights from memory and there are too few workgroups to keep it busy; the 64-row
      tile with its deeper run of loads (shape 4) streams faster, as long as the groups that take
      every row do not need many of those small tiles.  (With 128 experts there are workgroups
      enough: measured no gain.)
    * Else 128 rows a tile (shape 1), or 160 (shape 3, about a sixth dearer per tile) where that
      saves time: with groups of about 128 rows half of them need a second tile of 128, almost
      none a second one of 160.  The expected number of row tiles of each shape, group sizes
      taken as normal around tokens/groups, times ``col_tiles`` column tiles, runs on ``cus``
      compute units in whole rounds (a workgroup a unit): the fewer rounds, each at its tile's
      cost, win.  (Measured at widths of 4,096 to 6,144, 8 and 16 experts of 8,192 and 14,336:
      the choice by rounds was the faster tile in all eight products.)  Without ``col_tiles`` the
      row tiles alone are compared."""
    if groups <= 0 or tokens <= 0:
        return 1
    mean = tokens / groups
    sd = max(math.sqrt(tokens * (1.0 / groups) * (1.0 - 1.0 / groups)), 1e-6)
    if groups <= 32 and mean + 4.0 * sd <= 64.0 and whole_groups * -(-tokens // 64) <= 0.25 * groups:
        return 4

    def tiles(rows_per_tile):
        extra, k = 0.0, 1
        while k * rows_per_tile < mean + 6 * sd:
            extra += 0.5 * math.erfc((k * rows_per_tile + 0.5 - mean) / (sd * math.sqrt(2.0)))
            k += 1
        return groups * (1.0 + extra) + whole_groups * -(-tokens // rows_per_tile)
    if col_tiles > 0:
        cus = cus or hipops.cu_count()
        rounds = lambda rows_per_tile: math.ceil(tiles(rows_per_tile) * col_tiles / cus - 1e-9)
        return 3 if TILE_160_COST * rounds(160) < rounds(128) else 1
    return 3 if 1.17 * tiles(160) < tiles(128) else 1


def linear(x, w, y, *, glu=False, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, rows=None,
           max_rows=None, tile_shape=0, live_groups=0, ws=None):
    """y[r] = W . x[r] for ``rows`` rows (default: all of x; for a row list: its length).

    With ``glu`` the weight holds gate rows then up rows and y = silu(gate) * up.
    ``max_rows``: the most rows that one group can bring (default: ``rows``).
    ``tile_shape``: the prefill product's tile (``grouped_tile_shape``), 0 = the library's choice.
    ``live_groups``: a promise that at most this many groups hold rows (0: none).
    ``ws``: the workspace that temporaries (partial sums, widened rows) are taken from."""
    tiled = False
    if isinstance(w, Weight):
        w, tiled = w.data, w.tiled
    K = x.shape[-1]
    N = y.shape[-1]
    M = rows if rows is not None else x.shape[0]
    most = max_rows if max_rows is not None else M
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and x.stride(0) % 8 == 0:
        # few rows: the time is the weights' stream (a very tall matrix, the output table, is
        # streamed faster by the tiled kernel from 33 rows on)
        if most <= SKINNY_MAX_ROWS and not (tiled and most > 32 and offsets is None and N >= 65536):
            hipops.gemm_skinny(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                               a_scale=a_scale, y_rows=y_rows, glu=glu, max_rows=most, tiled=tiled,
                               live_groups=live_groups)
        elif tiled:
            plain = offsets is None and a_rows is None and a_scale is None and y_rows is None and not glu and tile_shape == 0
            runs = hipops.tiled_k_runs(M, N, K) if plain and M > 0 else 1
            part = _scratch(ws, (runs, M, N), torch.float32, x.device) if runs > 1 else None
            hipops.gemm_tiled(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows, a_scale=a_scale,
                              y_rows=y_rows, glu=glu, shape=tile_shape, part=part)
        else:
            hipops.gemm_mfma(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows, a_scale=a_scale,
                             y_rows=y_rows, glu=glu)
        return
    if tiled:
        raise hipops.KernelError("linear: a weight in operand order met an input that the MFMA products do not take")
    if w.dtype == torch.float32 and x.dtype != torch.float32:
        x32 = _widen(x, ws)
        if y.dtype == torch.float32:
            hipops.gemm_generic(x32, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                                a_scale=a_scale, y_rows=y_rows, glu=glu)
        else:
            y32 = _scratch(ws, y.shape, torch.float32, y.device)
            hipops.gemm_generic(x32, w, y32, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                                a_scale=a_scale, y_rows=y_rows, glu=glu)
            hipops.convert(y32, y)
        return
    hipops.gemm_generic(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows, a_scale=a_scale,
                        y_rows=y_rows, glu=glu)
