"""ctypes binding of the gfx950 kernel library: one Python function per entry point.

Arguments are torch tensors on the GPU; each wrapper checks device, dtype, contiguity and the
shapes that the kernel's indexing assumes before it launches, and raises ``KernelError`` with
the library's message when the library refuses a size.  There is no fallback: without the
library, or with a tensor that is not on the GPU, the call fails.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_long, c_float, c_void_p, c_size_t, c_char_p

import numpy as np
import torch

from . import build

F32, BF16 = 0, 1
VIS = build.visibility_codes()      # "full", "chunk", "window": name -> code


class KernelError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        l = build.load("hip")
        l.spite_hip_last_error.restype = c_char_p
        P, I, L, F = c_void_p, c_int, c_long, c_float
        sigs = {
            "spite_embed": [P, P, I, P, I, I, I, P],
            "spite_add_rmsnorm": [P, P, P, P, P, I, P, P, I, I, F, I, P, P, I, P],
            "spite_rope_kvwrite": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, I, I, F, I, I, I, P, P, I, P],
            "spite_router_top1": [P, P, P, P, P, I, I, I, P],
            "spite_moe_plan": [P, P, P, P, P, P, P, I, I, I, P],
            "spite_convert": [P, I, P, I, c_size_t, P],
            "spite_add_into": [P, P, c_size_t, P],
            "spite_randn_fill": [P, I, c_size_t, ctypes.c_ulonglong, ctypes.c_ulonglong, F, F, P],
            "spite_gemm_generic": [P, I, P, L, I, P, I, I, I, I, I, P, I, P, P, P, I, P],
            "spite_attn_generic": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, P],
            "spite_sample_rows": [P, I, I, I, P, P, P, P],
            "spite_filter_rows": [P, I, I, I, P, P, P, P],
            "spite_gemm_skinny": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, I, I, I, P],
            "spite_attn_decode": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, P],
            "spite_gemm_mfma": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, P],
            "spite_gemm_tiled": [P, I, P, L, P, I, I, I, I, I, P, I, P, P, P, I, I, P],
            "spite_gemm_tiled_split": [P, I, P, P, I, I, I, I, I, I, P, P],
            "spite_attn_prefill": [P, P, P, P, P, P, P, P, I, P, I, I, I, I, I, I, I, F, F, P, I, P],
            "spite_attn_prefill_splits": [P, I, I, I, L],
            "spite_argmax_rows": [P, I, I, I, P, P, P, P],
            "spite_stream_read": [P, c_size_t, P, I, P],
            "spite_mfma_loop": [P, I, I, F, P],
        }
        for name, args in sigs.items():
            fn = getattr(l, name)
            fn.argtypes = args
            fn.restype = c_int
        l.spite_attn_prefill_workspace.argtypes = [P, I, I, I, I, I]
        l.spite_attn_prefill_workspace.restype = c_size_t
        l.spite_cu_count.argtypes = []
        l.spite_cu_count.restype = c_int
        _lib = l
    return _lib


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"no kernel for dtype {dt}; the engine computes in float32 or bfloat16")


def _ptr(t, name, dtype=None, optional=False):
    if t is None:
        if optional:
            return None
        raise KernelError(f"{name}: missing tensor")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    return t.data_ptr()


def _check_pages(k_pages, v_pages, G, page_size, hd, what):
    """Key pages [n, G, page_size, hd]; value pages transposed, [n, G, hd, page_size]."""
    if (tuple(k_pages.shape[1:]) != (G, page_size, hd) or tuple(v_pages.shape[1:]) != (G, hd, page_size)
            or k_pages.shape[0] != v_pages.shape[0]):
        raise KernelError(f"{what}: key pages {tuple(k_pages.shape)}, value pages {tuple(v_pages.shape)} for "
                          f"G={G} page={page_size} hd={hd}")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check(rc, what):
    if rc != 0:
        raise KernelError(f"{what}: {lib().spite_hip_last_error().decode()}")


# --------------------------------------------------------------------------------------------
def embed(ids, table, h):
    """h[t,:] = table[ids[t],:] as fp32.  ids int32 [T], table [V,d], h fp32 [T,d]."""
    T, d = h.shape
    if ids.numel() != T or table.shape[1] != d:
        raise KernelError(f"embed: ids {tuple(ids.shape)}, table {tuple(table.shape)}, h {tuple(h.shape)}")
    _check(lib().spite_embed(_ptr(ids, "ids", torch.int32), _ptr(table, "table"), dtype_code(table.dtype),
                             _ptr(h, "h", torch.float32), T, d, table.shape[0], _stream()), "embed")


def add_rmsnorm_can_project(d: int) -> bool:
    """Whether ``add_rmsnorm`` forms projections of rows of this width (the row stays in LDS)."""
    return d * 4 <= 48 * 1024


def add_rmsnorm(h, w, eps, out=None, out32=None, d1=None, d2=None, rows=None, n_rows=None, write_h=True,
                proj=None, proj_out=None):
    """v = h[r] + d1[r] + d2[r] (stored back if write_h); out[i] = rmsnorm(v) * w with r =
    rows[i] or i.  h, d1, d2, out32 fp32; w fp32 [d]; out fp32 or bf16.  With ``proj`` ([P, d]
    fp32) also proj_out[i] = proj . (the normed row in fp32), [n, P] fp32: the same bits as
    ``router_top1`` gives for that row."""
    d = h.shape[-1]
    n = n_rows if n_rows is not None else (rows.numel() if rows is not None else h.shape[0])
    for name, t in (("d1", d1), ("d2", d2)):
        if t is not None and (t.shape[-1] != d or t.shape[0] < h.shape[0]):
            raise KernelError(f"add_rmsnorm: {name} {tuple(t.shape)} does not match h {tuple(h.shape)}")
    if w.numel() != d:
        raise KernelError(f"add_rmsnorm: weight of {w.numel()} for rows of {d}")
    for name, t in (("out", out), ("out32", out32)):
        if t is not None and (t.shape[-1] != d or t.shape[0] < n):
            raise KernelError(f"add_rmsnorm: {name} {tuple(t.shape)} is too small for {n} rows of {d}")
    if rows is None and n > h.shape[0]:
        raise KernelError("add_rmsnorm: more rows asked than h holds")
    P = 0
    if proj is not None:
        P = proj.shape[0]
        if proj.dim() != 2 or proj.shape[1] != d or proj_out is None or proj_out.dim() != 2 \
                or proj_out.shape[0] < n or proj_out.shape[1] != P:
            raise KernelError("add_rmsnorm: projection [P, d] with an output [rows, P]")
    _check(lib().spite_add_rmsnorm(
        _ptr(h, "h", torch.float32), _ptr(d1, "d1", torch.float32, True), _ptr(d2, "d2", torch.float32, True),
        _ptr(w, "w", torch.float32), _ptr(out, "out", None, True),
        dtype_code(out.dtype) if out is not None else F32, _ptr(out32, "out32", torch.float32, True),
        _ptr(rows, "rows", torch.int32, True), n, d, float(eps), int(write_h),
        _ptr(proj, "proj", torch.float32, True), _ptr(proj_out, "proj_out", torch.float32, True), P, _stream()),
        "add_rmsnorm")


def rope_kvwrite(qkv, q_out, k_pages, v_pages, positions, slot_map, inv_freq, H, G, hd, page_size, *,
                 use_rope, adjacent, use_norm, norm_eps, use_temp, floor_scale, attn_scale, write_kv=True,
                 kv_tiled=False, rotary_dim=None, norm_weight_q=None, norm_weight_k=None, norm_first=False):
    """Rotation, qk-norm and temperature of the fused projection's rows; keys and values go to
    their cache rows.  qkv [T,(H+2G)*hd]; q_out [T,H*hd]; key pages [n_pages, G, page_size, hd],
    value pages [n_pages, G, hd, page_size].  ``rotary_dim``: only the first so many elements of a
    head rotate (default: all); ``norm_weight_q`` / ``norm_weight_k`` (fp32 [hd]): the norm's
    weights (default: weightless); ``norm_first``: the norm comes before the rotation."""
    T = qkv.shape[0]
    if qkv.shape[1] != (H + 2 * G) * hd:
        raise KernelError(f"rope_kvwrite: qkv {tuple(qkv.shape)} for H={H} G={G} hd={hd}")
    if q_out.numel() < T * H * hd or positions.numel() < T:
        raise KernelError("rope_kvwrite: q_out or positions too small")
    if write_kv:
        if slot_map.numel() < T:
            raise KernelError("rope_kvwrite: slot map too small")
        _check_pages(k_pages, v_pages, G, page_size, hd, "rope_kvwrite")
    rot = hd if rotary_dim is None else int(rotary_dim)
    if hd % 2:
        raise KernelError(f"rope_kvwrite: head size {hd} must be even")
    if rot % 2 or not 0 < rot <= hd:
        raise KernelError(f"rope_kvwrite: {rot} rotating elements of a head of {hd}")
    if use_rope and inv_freq.numel() != rot // 2:
        raise KernelError("rope_kvwrite: frequency table does not match the rotating part of the head")
    for name, w in (("norm_weight_q", norm_weight_q), ("norm_weight_k", norm_weight_k)):
        if w is not None and (w.numel() != hd or not use_norm):
            raise KernelError(f"rope_kvwrite: {name} of {w.numel()} for heads of {hd} (norm {'on' if use_norm else 'off'})")
    dt = qkv.dtype
    _check(lib().spite_rope_kvwrite(
        _ptr(qkv, "qkv"), _ptr(q_out, "q_out", dt), _ptr(k_pages, "k_pages", dt, not write_kv),
        _ptr(v_pages, "v_pages", dt, not write_kv), dtype_code(dt), _ptr(positions, "positions", torch.int32),
        _ptr(slot_map, "slot_map", torch.int32, not write_kv), _ptr(inv_freq, "inv_freq", torch.float32, not use_rope),
        T, H, G, hd, page_size, int(use_rope), int(adjacent), int(use_norm), float(norm_eps), int(use_temp),
        int(floor_scale), float(attn_scale), int(write_kv), int(bool(kv_tiled)), rot,
        _ptr(norm_weight_q, "norm_weight_q", torch.float32, True), _ptr(norm_weight_k, "norm_weight_k", torch.float32, True),
        int(bool(norm_first)), _stream()), "rope_kvwrite")


def router_top1(x32, w_router, expert, weight, logits_out=None):
    """Top-1 sigmoid router on fp32 rows.  x32 [T,d], w_router fp32 [E,d]."""
    T, d = x32.shape
    E = w_router.shape[0]
    if w_router.shape[1] != d or expert.numel() < T or weight.numel() < T:
        raise KernelError("router_top1: shapes do not match")
    if logits_out is not None and logits_out.numel() < T * E:
        raise KernelError("router_top1: logits_out too small")
    _check(lib().spite_router_top1(_ptr(x32, "x32", torch.float32), _ptr(w_router, "w_router", torch.float32),
                                   _ptr(expert, "expert", torch.int32), _ptr(weight, "weight", torch.float32),
                                   _ptr(logits_out, "logits_out", torch.float32, True), T, d, E, _stream()),
           "router_top1")


def moe_plan(expert, weight, src, scale, dst, offsets, T, E, shared, logits=None):
    """Row list of the grouped products from the router's choice (see the kernel).  With
    ``logits`` ([T, E] fp32) the choice is made here and written to ``expert`` and ``weight``."""
    n = 2 * T if shared else T
    if src.numel() < n or scale.numel() < n or dst.numel() < n or offsets.numel() < E + 1 + int(bool(shared)):
        raise KernelError("moe_plan: output arrays too small")
    if expert.numel() < T or weight.numel() < T:
        raise KernelError("moe_plan: inputs too small")
    if logits is not None and (logits.dim() != 2 or logits.shape[0] < T or logits.shape[1] != E):
        raise KernelError(f"moe_plan: logits {tuple(logits.shape)} for {T} tokens and {E} experts")
    _check(lib().spite_moe_plan(_ptr(expert, "expert", torch.int32), _ptr(weight, "weight", torch.float32),
                                _ptr(logits, "logits", torch.float32, True), _ptr(src, "src", torch.int32), _ptr(scale, "scale", torch.float32),
                                _ptr(dst, "dst", torch.int32), _ptr(offsets, "offsets", torch.int32),
                                T, E, int(bool(shared)), _stream()), "moe_plan")


def convert(src, dst):
    if src.numel() != dst.numel():
        raise KernelError("convert: sizes differ")
    _check(lib().spite_convert(_ptr(src, "src"), dtype_code(src.dtype), _ptr(dst, "dst"), dtype_code(dst.dtype),
                               src.numel(), _stream()), "convert")


def add_into(h, d):
    """h += d, both fp32 and of one size (an increment of the residual stream beyond the two
    that a norm adds itself)."""
    if h.numel() != d.numel() or not h.is_contiguous() or not d.is_contiguous():
        raise KernelError(f"add_into: {tuple(h.shape)} and {tuple(d.shape)} must be contiguous and of one size")
    _check(lib().spite_add_into(_ptr(h, "h", torch.float32), _ptr(d, "d", torch.float32), h.numel(), _stream()), "add_into")


def randn_fill(t, seed: int, key: int, mean: float = 0.0, std: float = 1.0):
    """t[i] = mean + std * z(seed, key, i) with z standard normal: counter-based, so a tensor's
    numbers depend on the seed, its key and the element's index alone."""
    if not t.is_contiguous():
        raise KernelError("randn_fill: the tensor must be contiguous")
    _check(lib().spite_randn_fill(_ptr(t, "t"), dtype_code(t.dtype), t.numel(), int(seed) & ((1 << 64) - 1),
                                  int(key) & ((1 << 64) - 1), float(mean), float(std), _stream()), "randn_fill")


def gemm_generic(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None,
                 glu=False):
    """Y = A . W^T (see gemm_generic.hip).  a [rows,K]; w [groups, N or 2N, K] or [N or 2N, K];
    y [rows,N]."""
    if a.shape[-1] != K or y.shape[-1] != N:
        raise KernelError(f"gemm: a {tuple(a.shape)}, y {tuple(y.shape)} for N={N} K={K}")
    rows_w = 2 * N if glu else N
    if w.shape[-1] != K or w.shape[-2] != rows_w:
        raise KernelError(f"gemm: weight {tuple(w.shape)} for N={N} K={K} glu={glu}")
    groups_w = w.shape[0] if w.dim() == 3 else 1
    if offsets is not None:
        if groups_w < n_groups or offsets.numel() < n_groups + 1:
            raise KernelError("gemm: fewer weight groups or offsets than groups")
    if a_rows is None and a.shape[0] < M:
        raise KernelError("gemm: A has fewer rows than M")
    if y_rows is None and y.shape[0] < M:
        raise KernelError("gemm: Y has fewer rows than M")
    for name, t in (("a_rows", a_rows), ("a_scale", a_scale), ("y_rows", y_rows)):
        if t is not None and t.numel() < M:
            raise KernelError(f"gemm: {name} shorter than M")
    if w.dtype != a.dtype:
        raise KernelError(f"gemm: activations {a.dtype} against weights {w.dtype}")
    _check(lib().spite_gemm_generic(
        _ptr(a, "a"), a.stride(0) if a.dim() == 2 else K, _ptr(w, "w"), rows_w * K, dtype_code(a.dtype),
        _ptr(y, "y"), dtype_code(y.dtype), y.stride(0), M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups,
        _ptr(a_rows, "a_rows", torch.int32, True), _ptr(a_scale, "a_scale", torch.float32, True),
        _ptr(y_rows, "y_rows", torch.int32, True), int(glu), _stream()), "gemm")


def attn_generic(q, k_pages, v_pages, out, positions, seq_of_token, block_table, T, H, G, hd, page_size,
                 vis, span, scale, kv_tiled=False, softcap=0.0, slopes=None):
    """Attention over the paged cache, any mix of portions and single tokens.  q/out
    [T,H*hd]; block_table int32 [n_seqs, max_blocks].  ``kv_tiled``: the pages are in operand
    order (``kv_operand_order``).  Here and in the MFMA kernels: ``slopes`` (fp32 [H]) adds
    slopes[head] * (key position - query position) to the scaled scores; ``softcap`` > 0 then caps
    them smoothly, ``softcap * tanh(score / softcap)``, before the softmax."""
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attention: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attention")
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError("attention: metadata too small")
    dt = q.dtype
    _check(lib().spite_attn_generic(
        _ptr(q, "q"), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        dtype_code(dt), _ptr(positions, "positions", torch.int32), _ptr(seq_of_token, "seq_of_token", torch.int32),
        _ptr(block_table, "block_table", torch.int32), block_table.shape[1], T, H, G, hd, page_size,
        VIS[vis], int(span or 0), float(scale), float(softcap), _slopes(slopes, H), int(bool(kv_tiled)), _stream()), "attention")


def sample_rows(logits, temperature, uniform, out, n_rows=None):
    """out[r] = arg-max of row r (temperature[r] <= 0 or no temperatures) or the inverse-CDF
    draw with uniform[r].  logits fp32 [n,V]."""
    n = n_rows if n_rows is not None else logits.shape[0]
    if out.numel() < n or logits.shape[0] < n:
        raise KernelError("sample: too few rows")
    for name, t in (("temperature", temperature), ("uniform", uniform)):
        if t is not None and t.numel() < n:
            raise KernelError(f"sample: {name} shorter than the rows")
    _check(lib().spite_sample_rows(_ptr(logits, "logits", torch.float32), logits.stride(0), n, logits.shape[1],
                                   _ptr(temperature, "temperature", torch.float32, True),
                                   _ptr(uniform, "uniform", torch.float32, True),
                                   _ptr(out, "out", torch.int32), _stream()), "sample")


def filter_rows(work, params, pen_ids, pen_offsets):
    """The reference's filters on the rows of ``work`` (fp32 [n, V]) in place: repetition
    penalty, temperature, min-p, top-k, top-p (see sampling.hip).  ``params``: float64 [6, n]
    (on, temperature, ln(min_p), top_k, top_p, penalty); ``pen_ids`` int32, row r's distinct ids
    at ``pen_offsets[r] .. pen_offsets[r+1]`` (int32 [n+1]); the caller keeps the ids inside [0, V)."""
    n = work.shape[0]
    if params.dtype != torch.float64 or tuple(params.shape) != (6, n) or not params.is_contiguous():
        raise KernelError(f"filter: params {tuple(params.shape)} {params.dtype} for {n} rows")
    if pen_offsets.numel() != n + 1:
        raise KernelError(f"filter: {pen_offsets.numel()} offsets for {n} rows")
    _check(lib().spite_filter_rows(_ptr(work, "work", torch.float32), work.stride(0), n, work.shape[1],
                                   _ptr(params, "params", torch.float64), _ptr(pen_ids, "pen_ids", torch.int32, True),
                                   _ptr(pen_offsets, "pen_offsets", torch.int32), _stream()), "filter")


def _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, what):
    if a.shape[-1] != K or y.shape[-1] != N:
        raise KernelError(f"{what}: a {tuple(a.shape)}, y {tuple(y.shape)} for N={N} K={K}")
    rows_w = 2 * N if glu else N
    if w.shape[-1] != K or w.shape[-2] != rows_w:
        raise KernelError(f"{what}: weight {tuple(w.shape)} for N={N} K={K} glu={glu}")
    groups_w = w.shape[0] if w.dim() == 3 else 1
    if offsets is not None and (groups_w < n_groups or offsets.numel() < n_groups + 1):
        raise KernelError(f"{what}: fewer weight groups or offsets than groups")
    if a_rows is None and a.shape[0] < M:
        raise KernelError(f"{what}: A has fewer rows than M")
    if y_rows is None and y.shape[0] < M:
        raise KernelError(f"{what}: Y has fewer rows than M")
    for name, t in (("a_rows", a_rows), ("a_scale", a_scale), ("y_rows", y_rows)):
        if t is not None and t.numel() < M:
            raise KernelError(f"{what}: {name} shorter than M")
    return rows_w


def gemm_skinny(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None,
                glu=False, max_rows=None, variant=0, tiled=False, live_groups=0):
    """Weight-streaming bf16 product for few rows (see gemm_skinny.hip); arguments as gemm_generic.
    ``max_rows``: the most rows a group can bring (default M).  ``tiled``: w is in MFMA operand
    order (``operand_order``).  ``live_groups``: a promise that at most this many groups hold rows
    (0: none); row tiles beyond what that allows are not launched."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_skinny")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_skinny: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    _check(lib().spite_gemm_skinny(
        _ptr(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), int(glu),
        int(max_rows if max_rows is not None else M), int(variant), int(bool(tiled)), int(live_groups), _stream()),
        "gemm_skinny")


def kv_tiled_ok(dtype, hd, page_size) -> bool:
    """Whether cache pages of this kind are kept in MFMA operand order."""
    return dtype == torch.bfloat16 and hd % 32 == 0 and page_size % 32 == 0


def kv_operand_order(k_pages, v_pages):
    """Copies of row-major pages (keys [n, G, page_size, hd], values transposed [n, G, hd,
    page_size]) in the operand order that the MFMA attention kernels read; same shapes.
    Keys: blocks of 32 keys, two tiles of 16 rows (row r of tile tt = key (r/4)*8 + tt*4 + r%4),
    hd/32 chunks each, a tile's [16 rows][32 elements] stored as [4 q][16 r][8 e].  Values:
    per block of 32 keys, tiles of 16 head elements, [16 rows][32 keys] stored the same way."""
    n, G, ps, hd = k_pages.shape
    if ps % 32 or hd % 32:
        raise KernelError(f"operand order needs page size {ps} and head size {hd} to be multiples of 32")
    # key offset w = 8a + 4tt + i  ->  row r = 4a + i of tile tt; element c = 32cc + 8q + e
    k = k_pages.reshape(n, G, ps // 32, 4, 2, 4, hd // 32, 4, 8)          # b, a, tt, i, cc, q, e
    k = k.permute(0, 1, 2, 4, 6, 7, 3, 5, 8)                                # b, tt, cc, q, a, i, e
    # head element c = 16dt + r, key offset = 32b + 8q + e
    v = v_pages.reshape(n, G, hd // 16, 16, ps // 32, 4, 8)                # dt, r, b, q, e
    v = v.permute(0, 1, 4, 2, 5, 3, 6)                                      # b, dt, q, r, e
    return k.contiguous().view(n, G, ps, hd), v.contiguous().view(n, G, hd, ps)


def attn_decode_workspace(T, H, hd, n_splits) -> int:
    """Bytes of scratch that attn_decode needs."""
    return T * H * n_splits * (hd + 2) * 4


def attn_decode(q, k_pages, v_pages, out, workspace, positions, seq_of_token, block_table, T, H, G, hd,
                page_size, vis, span, scale, n_splits, softcap=0.0, slopes=None):
    """Split-KV decode attention on MFMA (bf16; head sizes 64 and 128; pages of a multiple of 32
    keys, in operand order): every row of q is one query against its request's cache."""
    if q.dtype != torch.bfloat16:
        raise KernelError(f"attn_decode: bfloat16 only, got {q.dtype}")
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attn_decode: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attn_decode")
    if block_table.dim() != 2 or positions.numel() < T or seq_of_token.numel() < T:
        raise KernelError("attn_decode: metadata too small")
    if workspace.numel() * workspace.element_size() < attn_decode_workspace(T, H, hd, n_splits):
        raise KernelError("attn_decode: workspace too small")
    dt = torch.bfloat16
    _check(lib().spite_attn_decode(
        _ptr(q, "q", dt), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        _ptr(workspace, "workspace"), _ptr(positions, "positions", torch.int32),
        _ptr(seq_of_token, "seq_of_token", torch.int32), _ptr(block_table, "block_table", torch.int32),
        block_table.shape[1], T, H, G, hd, page_size, VIS[vis], int(span or 0), float(scale), float(softcap),
        _slopes(slopes, H), int(n_splits), _stream()), "attn_decode")


def gemm_mfma(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, glu=False,
              shape=0):
    """Tiled bf16 MFMA product for many rows (see gemm_mfma.hip); arguments as gemm_generic."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_mfma")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_mfma: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    _check(lib().spite_gemm_mfma(
        _ptr(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), int(glu),
        int(shape), _stream()), "gemm_mfma")


def operand_order(w: torch.Tensor) -> torch.Tensor:
    """A copy of the matrices ``w[..., N, K]`` (N % 16 == 0, K % 64 == 0) in MFMA operand order:
    tiles of 16 rows x 32 k, tile (i, j) at ((i * K/32) + j) * 512 elements, inside it
    W[16i + r][32j + 8q + e] at (q*16 + r) * 8 + e.  Shape and dtype stay as they are."""
    *lead, N, K = w.shape
    if N % 16 or K % 64:
        raise KernelError(f"operand order needs rows a multiple of 16 and columns of 64, got {N} x {K}")
    n = len(lead)
    t = w.reshape(*lead, N // 16, 16, K // 32, 4, 8).permute(*range(n), n, n + 2, n + 3, n + 1, n + 4)
    return t.contiguous().view(*lead, N, K)


def tiled_k_runs(M: int, N: int, K: int) -> int:
    """Into how many runs the tiled product cuts its sum over k: with tiles of 128 rows x 512
    columns for fewer than half of the chip's CUs, those are not filled, and a run keeps at least
    four steps of 64 k."""
    cus = cu_count()
    tiles = -(-M // 128) * -(-N // 512)
    steps = K // 64
    runs = min(8, cus // max(tiles, 1), steps // 4)
    while runs > 1 and -(-steps // runs) * (runs - 1) >= steps:      # no run may be empty
        runs -= 1
    return runs if tiles < cus // 2 and runs > 1 else 1


_cu_count = None


def cu_count() -> int:
    """Compute units of the current GPU, as the library counts them."""
    global _cu_count
    if _cu_count is None:
        _cu_count = int(lib().spite_cu_count())
    return _cu_count


def gemm_tiled(a, w, y, M, N, K, *, offsets=None, n_groups=1, a_rows=None, a_scale=None, y_rows=None, glu=False,
               shape=0, part=None):
    """Tiled bf16 MFMA product for many rows over weights in operand order (``operand_order``;
    see gemm_tiled.hip); arguments as gemm_generic.  ``part`` (fp32 ``[runs, M, N]``, plain
    products only): the sum over k is cut into ``runs`` runs, each a workgroup of its own, whose
    partial sums a second kernel adds: for few tiles (a short prompt against a narrow matrix),
    see ``tiled_k_runs``."""
    rows_w = _gemm_checks(a, w, y, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, "gemm_tiled")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_tiled: bfloat16 operands only, got {a.dtype} and {w.dtype}")
    if part is not None:
        if not (offsets is None and a_rows is None and a_scale is None and y_rows is None and not glu and shape == 0):
            raise KernelError("gemm_tiled: partial sums are for plain products only")
        if part.dim() != 3 or part.shape[1] != M or part.shape[2] != N or part.shape[0] < 2 or part.shape[0] > 32 \
                or part.shape[0] * 2 > K // 64:
            raise KernelError(f"gemm_tiled: partial sums {tuple(part.shape)} for M={M} N={N} K={K}")
        _check(lib().spite_gemm_tiled_split(_ptr(a, "a"), a.stride(0), _ptr(w, "w"), _ptr(y, "y"), dtype_code(y.dtype),
                                            y.stride(0), M, N, K, part.shape[0], _ptr(part, "part", torch.float32),
                                            _stream()), "gemm_tiled")
        return
    _check(lib().spite_gemm_tiled(
        _ptr(a, "a"), a.stride(0), _ptr(w, "w"), rows_w * K, _ptr(y, "y"), dtype_code(y.dtype), y.stride(0),
        M, N, K, _ptr(offsets, "offsets", torch.int32, True), n_groups, _ptr(a_rows, "a_rows", torch.int32, True),
        _ptr(a_scale, "a_scale", torch.float32, True), _ptr(y_rows, "y_rows", torch.int32, True), int(glu),
        int(shape), _stream()), "gemm_tiled")


def attn_prefill_splits(counts, H, G, max_keys) -> int:
    """Into how many splits the prefill kernel's tiles of this step are best cut (1: none), for
    ``counts`` query tokens per request and at most ``max_keys`` keys read by a query."""
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    return int(lib().spite_attn_prefill_splits(counts.ctypes.data, int(counts.size), H, G, int(max_keys)))


def attn_prefill_workspace(counts, H, G, hd, n_splits) -> int:
    """Bytes of fp32 scratch that ``attn_prefill`` needs for ``n_splits`` > 1 (none for 1)."""
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    return int(lib().spite_attn_prefill_workspace(counts.ctypes.data, int(counts.size), H, G, hd, int(n_splits)))


def attn_prefill(q, k_pages, v_pages, out, positions, cu_seqlens, counts, block_table,
                 H, G, hd, page_size, vis, span, scale, n_splits=1, scratch=None, softcap=0.0, slopes=None):
    """Prefill attention on MFMA (bf16; head sizes 64 and 128; pages of a multiple of 32 keys, in
    operand order).
    ``counts``: the number of query tokens of every request of the step, on the host, in the
    order of ``cu_seqlens`` (their running sum, on the device) and of the block table's rows.
    ``n_splits`` > 1 deals every tile's keys to that many workgroups; ``scratch`` (fp32,
    ``attn_prefill_workspace`` bytes) then holds their partial results.
    ``slopes`` (fp32 [H] or None): a bias slopes[head] * (key position - query position) on the
    scaled scores, before the cap."""
    if q.dtype != torch.bfloat16:
        raise KernelError(f"attn_prefill: bfloat16 only, got {q.dtype}")
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    n_seqs = int(counts.size)
    T = int(counts.sum())
    if q.numel() < T * H * hd or out.numel() < T * H * hd:
        raise KernelError("attn_prefill: q or out too small")
    _check_pages(k_pages, v_pages, G, page_size, hd, "attn_prefill")
    if block_table.dim() != 2 or block_table.shape[0] < n_seqs or positions.numel() < T:
        raise KernelError("attn_prefill: metadata too small")
    if cu_seqlens.numel() < n_seqs + 1:
        raise KernelError("attn_prefill: cu_seqlens shorter than the requests of the step")
    n_splits = int(n_splits)
    if n_splits > 1 and (scratch is None or scratch.numel() * 4 < attn_prefill_workspace(counts, H, G, hd, n_splits)):
        raise KernelError(f"attn_prefill: {n_splits} splits need {attn_prefill_workspace(counts, H, G, hd, n_splits)} bytes of scratch")
    dt = torch.bfloat16
    _check(lib().spite_attn_prefill(
        _ptr(q, "q", dt), _ptr(k_pages, "k_pages", dt), _ptr(v_pages, "v_pages", dt), _ptr(out, "out", dt),
        _ptr(scratch, "scratch", torch.float32) if n_splits > 1 else None,
        _ptr(positions, "positions", torch.int32), _ptr(cu_seqlens, "cu_seqlens", torch.int32),
        counts.ctypes.data, n_seqs, _ptr(block_table, "block_table", torch.int32), block_table.shape[1],
        H, G, hd, page_size, VIS[vis], int(span or 0), float(scale), float(softcap), _slopes(slopes, H), n_splits,
        _stream()), "attn_prefill")


def _slopes(slopes, H):
    if slopes is None:
        return None
    if slopes.numel() != H:
        raise KernelError(f"score slopes: {slopes.numel()} values for {H} query heads")
    return _ptr(slopes, "slopes", torch.float32)


def argmax_rows(logits, out, scratch_v, scratch_i, n_rows=None):
    """out[r] = index of the largest logit of row r, the lowest among equals.  Scratch: 32 floats
    and 32 ints per row."""
    n = n_rows if n_rows is not None else logits.shape[0]
    if out.numel() < n or logits.shape[0] < n or scratch_v.numel() < 32 * n or scratch_i.numel() < 32 * n:
        raise KernelError("argmax: outputs or scratch too small")
    _check(lib().spite_argmax_rows(_ptr(logits, "logits", torch.float32), logits.stride(0), n, logits.shape[1],
                                   _ptr(scratch_v, "scratch_v", torch.float32), _ptr(scratch_i, "scratch_i", torch.int32),
                                   _ptr(out, "out", torch.int32), _stream()), "argmax")


def stream_read(t, out):
    """Reads the tensor ``t`` once with non-temporal loads, one contiguous piece per workgroup;
    ``out`` (fp32, eight elements per workgroup) receives sums that keep the loads alive.  For
    measuring the memory's read bandwidth."""
    nbytes = t.numel() * t.element_size()
    if out.numel() < 8:
        raise KernelError("stream_read: out holds eight floats per workgroup")
    _check(lib().spite_stream_read(_ptr(t, "t"), nbytes - nbytes % 16, _ptr(out, "out", torch.float32), out.numel() // 8,
                                   _stream()), "stream_read")


def mfma_loop(out, steps, gain):
    """Runs ``out.numel()`` workgroups of eight waves, every wave ``steps`` times 32 MFMA 16x16x32 on
    operands in registers (pseudo-random values scaled by ``gain``; 0: all zero): the matrix units'
    rate with nothing else moving.  Returns the flops done."""
    _check(lib().spite_mfma_loop(_ptr(out, "out", torch.float32), out.numel(), int(steps), float(gain), _stream()), "mfma_loop")
    return out.numel() * 8 * int(steps) * 32 * 16384
