"""Matrix products of the parts: picks the kernel for the dtypes and shapes at hand.

``Y = X . W^T`` with W ``[out, in]``; the grouped form walks a row list (see
``gemm_generic.hip``).  A weight that stayed in 32-bit inside a bfloat16 run is multiplied in
32-bit: the activations are widened for that product.
"""
from __future__ import annotations

import torch

from ..csrc import hipops


def _widen(x):
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    hipops.convert(x, y)
    return y


SKINNY_MAX_ROWS = 64


def linear(x, w, y, *, glu=False, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, rows=None,
           max_rows=None):
    """y[r] = W . x[r] for ``rows`` rows (default: all of x; for a row list: its length).

    With ``glu`` the weight holds gate rows then up rows and y = silu(gate) * up.
    ``max_rows``: the most rows that one group can bring (default: ``rows``)."""
    K = x.shape[-1]
    N = y.shape[-1]
    M = rows if rows is not None else x.shape[0]
    most = max_rows if max_rows is not None else M
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and x.stride(0) % 8 == 0:
        if most <= SKINNY_MAX_ROWS:      # few rows: the time is the weights' stream
            hipops.gemm_skinny(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                               a_scale=a_scale, y_rows=y_rows, glu=glu, max_rows=most)
        else:
            hipops.gemm_mfma(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows, a_scale=a_scale,
                             y_rows=y_rows, glu=glu)
        return
    if w.dtype == torch.float32 and x.dtype != torch.float32:
        x32 = _widen(x)
        if y.dtype == torch.float32:
            hipops.gemm_generic(x32, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                                a_scale=a_scale, y_rows=y_rows, glu=glu)
        else:
            y32 = torch.empty(y.shape, dtype=torch.float32, device=y.device)
            hipops.gemm_generic(x32, w, y32, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows,
                                a_scale=a_scale, y_rows=y_rows, glu=glu)
            hipops.convert(y32, y)
        return
    hipops.gemm_generic(x, w, y, M, N, K, offsets=offsets, n_groups=n_groups, a_rows=a_rows, a_scale=a_scale,
                        y_rows=y_rows, glu=glu)
