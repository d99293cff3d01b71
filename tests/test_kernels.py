"""Each kernel alone against a plain PyTorch reference in float64, at sizes other than the
tiny models': widths and vocabularies that are no power of two, head sizes in steps of 8,
any number of heads and groups, page edges."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama4 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from spite_amd.csrc import hipops
    return hipops


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol_for(dtype, ref):
    # fp32: accumulation noise; bf16: one rounding of the result (2^-9 relative) plus that
    return (2e-5 if dtype == torch.float32 else 6e-3) * max(float(ref.abs().max()), 1e-6)


# ------------------------------------------------------------------ embedding, norm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    table = rnd(301, 72, dtype=dtype)
    ids = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32, device=DEV)
    h = torch.empty(5, 72, dtype=torch.float32, device=DEV)
    ops().embed(ids, table, h)
    assert torch.equal(h, table[ids.long()].float())


@pytest.mark.parametrize("d", [40, 96, 1000, 5120])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm(d, out_dtype):
    T = 7
    h, d1, d2, w = rnd(T, d), rnd(T, d, seed=1), rnd(T, d, seed=2), rnd(d, seed=3) + 1.0
    ref_h = h.double() + d1.double() + d2.double()
    ref = F.rms_norm(ref_h, (d,), w.double(), 1e-6)
    out = torch.empty(T, d, dtype=out_dtype, device=DEV)
    out32 = torch.empty(T, d, dtype=torch.float32, device=DEV)
    hh = h.clone()
    ops().add_rmsnorm(hh, w, 1e-6, out=out, out32=out32, d1=d1, d2=d2)
    assert (hh.double() - ref_h).abs().max() < 1e-6
    assert (out32.double() - ref).abs().max() < tol_for(torch.float32, ref)
    assert (out.double() - ref).abs().max() < tol_for(out_dtype, ref)
    # chosen rows only, h untouched
    rows = torch.tensor([6, 2], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, d, dtype=torch.float32, device=DEV)
    hh = h.clone()
    ops().add_rmsnorm(hh, w, 1e-6, out=out2, d1=d1, rows=rows, write_h=False)
    ref2 = F.rms_norm(h.double() + d1.double(), (d,), w.double(), 1e-6)[[6, 2]]
    assert torch.equal(hh, h) and (out2.double() - ref2).abs().max() < tol_for(torch.float32, ref2)


# ------------------------------------------------------------------ rotation and cache write
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,hd,adjacent,norm,temp", [(4, 2, 16, False, True, False), (6, 3, 24, False, False, True),
                                                       (5, 1, 64, True, True, True), (8, 8, 128, False, True, False),
                                                       (2, 1, 256, False, True, False)])
@pytest.mark.parametrize("T", [11, 300])
def test_rope_kvwrite(dtype, H, G, hd, adjacent, norm, temp, T):
    ps, n_pages = 4, 9 if T == 11 else 80
    qkv = rnd(T, (H + 2 * G) * hd, dtype=dtype)
    if T == 11:
        pos = torch.tensor([3, 4, 5, 0, 1, 2, 3, 40, 41, 42, 7], dtype=torch.int32, device=DEV)
        slots = torch.tensor([5, 6, 7, 12, 13, 14, 15, 0, 1, 2, 35], dtype=torch.int32, device=DEV)
    else:                                          # many tokens: the kernel's long workgroups
        g = torch.Generator().manual_seed(T)
        pos = (torch.arange(T) % 57).to(torch.int32).to(DEV)
        slots = torch.randperm(n_pages * ps, generator=g)[:T].to(torch.int32).to(DEV)
    inv = plain.rope_inv_freq(hd, 10000.0, None).to(torch.float32).to(DEV)
    q = torch.empty(T, H * hd, dtype=dtype, device=DEV)
    kp = torch.zeros(n_pages, G, ps, hd, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, G, hd, ps, dtype=dtype, device=DEV)          # values are kept transposed
    ops().rope_kvwrite(qkv, q, kp, vp, pos, slots, inv, H, G, hd, ps, use_rope=True, adjacent=adjacent, use_norm=norm,
                       norm_eps=1e-5, use_temp=temp, floor_scale=4, attn_scale=0.1)
    x = qkv.double().cpu()
    qq, kk, vv = (x[:, :H * hd].view(T, H, hd), x[:, H * hd:(H + G) * hd].view(T, G, hd), x[:, (H + G) * hd:].view(T, G, hd))
    pc = pos.cpu()
    pairing = "adjacent" if adjacent else "half"
    rq, rk = plain.apply_rope(qq, pc, inv.double().cpu(), pairing), plain.apply_rope(kk, pc, inv.double().cpu(), pairing)
    if norm:
        rq, rk = plain.qk_l2_norm(rq, 1e-5), plain.qk_l2_norm(rk, 1e-5)
    if temp:
        rq = rq * plain.attn_temperature(pc, 4, 0.1)[:, None, None]
    tol = tol_for(dtype, rq) * (4 if dtype == torch.float32 else 1)
    assert (q.double().cpu().view(T, H, hd) - rq).abs().max() < tol
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert (kp[page, :, off].double().cpu() - rk[t]).abs().max() < tol
        assert torch.equal(vp[page, :, :, off].cpu().double(), vv[t])
    if ops().kv_tiled_ok(dtype, hd, 32):       # the same rows into pages of 32 in operand order
        kp32 = torch.zeros(n_pages, G, 32, hd, dtype=dtype, device=DEV)
        vp32 = torch.zeros(n_pages, G, hd, 32, dtype=dtype, device=DEV)
        kpt, vpt, q2 = torch.zeros_like(kp32), torch.zeros_like(vp32), torch.empty_like(q)
        slots32 = (slots // ps) * 32 + ((slots % ps) * 9 + (slots // ps)) % 32        # spread over the page's offsets
        for tiled, (a, b) in ((False, (kp32, vp32)), (True, (kpt, vpt))):
            ops().rope_kvwrite(qkv, q2, a, b, pos, slots32, inv, H, G, hd, 32, use_rope=True, adjacent=adjacent,
                               use_norm=norm, norm_eps=1e-5, use_temp=temp, floor_scale=4, attn_scale=0.1, kv_tiled=tiled)
            assert torch.equal(q2, q)
        want_k, want_v = ops().kv_operand_order(kp32, vp32)
        assert float(kp32.abs().sum()) > 0 and torch.equal(kpt, want_k) and torch.equal(vpt, want_v)
    written = {(int(s) // ps, int(s) % ps) for s in slots.cpu()}
    for p in range(n_pages):
        for o in range(ps):
            if (p, o) not in written:
                assert float(kp[p, :, o].abs().sum()) == 0 and float(vp[p, :, :, o].abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,hd,rot,adjacent,weighted,first", [
    (4, 2, 64, 32, False, True, True),      # half of the head rotates; weighted norm before the rotation
    (3, 1, 48, 16, True, True, False),      # adjacent pairs, a third rotates; weighted norm after it
    (6, 2, 128, 128, False, True, True),    # the whole head, weighted, norm first
    (2, 2, 32, 8, False, False, True),      # weightless norm first: the same numbers as norm after (rotation keeps lengths)
])
def test_rope_kvwrite_with_part_of_the_head_rotating_and_a_weighted_norm_before_or_after(dtype, H, G, hd, rot, adjacent, weighted, first):
    T, ps, n_pages = 37, 8, 6
    qkv = rnd(T, (H + 2 * G) * hd, dtype=dtype, seed=3)
    pos = ((torch.arange(T) * 7) % 50).to(torch.int32).to(DEV)
    slots = torch.randperm(n_pages * ps, generator=torch.Generator().manual_seed(1))[:T].to(torch.int32).to(DEV)
    inv = plain.rope_inv_freq(rot, 10000.0, None).to(torch.float32).to(DEV)
    wq, wk = (rnd(hd, seed=5) * 0.3 + 1.0, rnd(hd, seed=6) * 0.3 + 1.0) if weighted else (None, None)
    q = torch.empty(T, H * hd, dtype=dtype, device=DEV)
    kp = torch.zeros(n_pages, G, ps, hd, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, G, hd, ps, dtype=dtype, device=DEV)
    ops().rope_kvwrite(qkv, q, kp, vp, pos, slots, inv, H, G, hd, ps, use_rope=True, adjacent=adjacent, use_norm=True,
                       norm_eps=1e-5, use_temp=False, floor_scale=1, attn_scale=0.0, rotary_dim=rot,
                       norm_weight_q=wq, norm_weight_k=wk, norm_first=first)
    x = qkv.double().cpu()
    qq, kk = x[:, :H * hd].view(T, H, hd), x[:, H * hd:(H + G) * hd].view(T, G, hd)
    pc, pairing = pos.cpu(), "adjacent" if adjacent else "half"

    def rotate(v):        # the first `rot` elements as a head of that size, the rest untouched
        out = v.clone()
        out[..., :rot] = plain.apply_rope(v[..., :rot], pc, inv.double().cpu(), pairing)
        return out

    def norm(v, w):
        y = plain.rms_norm(v, None, 1e-5)
        return y if w is None else y * w.double().cpu()
    want_q, want_k = (rotate(norm(qq, wq)), rotate(norm(kk, wk))) if first else (norm(rotate(qq), wq), norm(rotate(kk), wk))
    tol = tol_for(dtype, want_q) * (4 if dtype == torch.float32 else 1.5)
    assert (q.double().cpu().view(T, H, hd) - want_q).abs().max() < tol
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert (kp[page, :, off].double().cpu() - want_k[t]).abs().max() < tol
    if ops().kv_tiled_ok(dtype, hd, 32):       # the same rows into pages of 32, row-major and in operand order
        kp32, vp32 = torch.zeros(n_pages, G, 32, hd, dtype=dtype, device=DEV), torch.zeros(n_pages, G, hd, 32, dtype=dtype, device=DEV)
        kpt, vpt, q2 = torch.zeros_like(kp32), torch.zeros_like(vp32), torch.empty_like(q)
        slots32 = (slots // ps) * 32 + ((slots % ps) * 9 + (slots // ps)) % 32
        for tiled, (a, b) in ((False, (kp32, vp32)), (True, (kpt, vpt))):
            ops().rope_kvwrite(qkv, q2, a, b, pos, slots32, inv, H, G, hd, 32, use_rope=True, adjacent=adjacent, use_norm=True,
                               norm_eps=1e-5, use_temp=False, floor_scale=1, attn_scale=0.0, rotary_dim=rot,
                               norm_weight_q=wq, norm_weight_k=wk, norm_first=first, kv_tiled=tiled)
            assert torch.equal(q2, q)
        want_kt, want_vt = ops().kv_operand_order(kp32, vp32)
        assert float(kp32.abs().sum()) > 0 and torch.equal(kpt, want_kt) and torch.equal(vpt, want_vt)
        for t in range(T):
            page, off = int(slots32[t]) // 32, int(slots32[t]) % 32
            assert (kp32[page, :, off].double().cpu() - want_k[t]).abs().max() < tol
    # a wrong order of norm and rotation shows where the weights are not all alike
    if weighted:
        other_q = norm(rotate(qq), wq) if first else rotate(norm(qq, wq))
        assert (other_q - want_q).abs().max() > 20 * tol


def test_rope_kvwrite_refuses_odd_sizes():
    from spite_amd.csrc.hipops import KernelError
    z = torch.zeros(1, 3 * 15, device=DEV)
    with pytest.raises(KernelError, match="even"):
        ops().rope_kvwrite(z, torch.zeros(1, 15, device=DEV), torch.zeros(1, 1, 4, 15, device=DEV),
                           torch.zeros(1, 1, 15, 4, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                           torch.zeros(1, dtype=torch.int32, device=DEV), None, 1, 1, 15, 4, use_rope=False,
                           adjacent=False, use_norm=False, norm_eps=1e-5, use_temp=False, floor_scale=1, attn_scale=0.0)


# ------------------------------------------------------------------ products
def gemm_reference(a, w, M, N, K, offsets=None, a_rows=None, a_scale=None, y_rows=None, glu=False, n_out_rows=None):
    a64, w64 = a.double().cpu(), w.double().cpu()
    out = torch.zeros(n_out_rows or M, N, dtype=torch.float64)
    groups = [(0, M, 0)] if offsets is None else [(int(offsets[g]), int(offsets[g + 1]), g) for g in range(len(offsets) - 1)]
    for b, e, g in groups:
        for s in range(b, e):
            x = a64[int(a_rows[s]) if a_rows is not None else s]
            if a_scale is not None:
                x = x * float(a_scale[s])
            wg = w64[g] if w64.dim() == 3 else w64
            y = wg @ x
            if glu:
                y = F.silu(y[:N]) * y[N:]
            out[int(y_rows[s]) if y_rows is not None else s] = y
    return out


GEMM_SHAPES = [(1, 48, 64), (7, 100, 264), (16, 130, 1032), (33, 96, 96), (64, 72, 520), (5, 202, 144)]


def run_gemm(fn, dtype, out_dtype, M, N, K, glu=False, grouped=False, groups=5, **kw):
    E = groups if grouped else 1
    a = rnd(M + 3, K, dtype=dtype, scale=0.5)
    w = rnd(*((E,) if grouped else ()), (2 * N if glu else N), K, dtype=dtype, seed=1, scale=0.5)
    args = dict(glu=glu)
    n_out = M
    if grouped:
        g = torch.Generator().manual_seed(M)
        cuts = sorted(torch.randint(0, M + 1, (E - 1,), generator=g).tolist())
        offsets = torch.tensor([0] + cuts + [M], dtype=torch.int32)
        a_rows = torch.randint(0, M + 3, (M,), generator=g).to(torch.int32)
        a_scale = torch.rand(M, generator=g) + 0.5
        y_rows = torch.randperm(M + 2, generator=g)[:M].to(torch.int32)
        n_out = M + 2
        args.update(offsets=offsets.to(DEV), n_groups=E, a_rows=a_rows.to(DEV), a_scale=a_scale.to(DEV), y_rows=y_rows.to(DEV))
        ref = gemm_reference(a, w, M, N, K, offsets, a_rows, a_scale, y_rows, glu, n_out)
    else:
        ref = gemm_reference(a, w, M, N, K, glu=glu)
    y = torch.zeros(n_out, N, dtype=out_dtype, device=DEV)
    fn(a, w, y, M, N, K, **args, **kw)
    err = (y.double().cpu() - ref).abs().max()
    assert err < tol_for(out_dtype, ref), (err, float(ref.abs().max()))


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("glu,grouped", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_generic(M, N, K, dtype, out_dtype, glu, grouped):
    if K % 8:
        pytest.skip("shape list is shared with the MFMA kernels")
    run_gemm(ops().gemm_generic, dtype, out_dtype, M, N, K, glu, grouped)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + [(3, 40, 8), (12, 16, 4104)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("glu,grouped", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("variant", [2, 3, 4, 6, 7, 8, 9, 10])
def test_gemm_skinny(M, N, K, out_dtype, glu, grouped, variant):
    run_gemm(ops().gemm_skinny, torch.bfloat16, out_dtype, M, N, K, glu, grouped, variant=variant)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + [(200, 300, 264), (128, 128, 64), (130, 70, 1032), (257, 129, 72)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("glu,grouped", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_mfma(M, N, K, out_dtype, glu, grouped):
    run_gemm(ops().gemm_mfma, torch.bfloat16, out_dtype, M, N, K, glu, grouped)


# weights in MFMA operand order: rows a multiple of 16, columns of 64
TILED_SHAPES = [(1, 48, 64), (7, 112, 320), (16, 144, 1088), (64, 80, 512), (33, 528, 192)]


@pytest.mark.parametrize("M,N,K", TILED_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("glu,grouped", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("variant", [2, 3, 4, 6, 7, 8, 9, 10])
def test_gemm_skinny_over_operand_order(M, N, K, out_dtype, glu, grouped, variant):
    def fn(a, w, y, *args, **kw):
        ops().gemm_skinny(a, ops().operand_order(w), y, *args, tiled=True, **kw)
    run_gemm(fn, torch.bfloat16, out_dtype, M, N, K, glu, grouped, variant=variant)


@pytest.mark.parametrize("M,N,K", TILED_SHAPES + [(200, 304, 256), (130, 160, 1024), (257, 528, 192), (520, 1040, 128),
                                                  (300, 64, 448)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("glu,grouped", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", [1, 2, 3, 4, 5])
def test_gemm_tiled(M, N, K, out_dtype, glu, grouped, shape):
    def fn(a, w, y, *args, **kw):
        ops().gemm_tiled(a, ops().operand_order(w), y, *args, **kw)
    run_gemm(fn, torch.bfloat16, out_dtype, M, N, K, glu, grouped, shape=shape)


@pytest.mark.parametrize("M,N,K", [(200, 304, 256), (97, 528, 192), (520, 1040, 128), (2048, 1024, 128)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_tiled_with_rows_in_tiles_of_96(M, N, K, out_dtype):
    """The tile that a plain product takes where its 128-row tiles would leave CUs without one: the
    same bits as the 128-row tile (the sum over k runs in the same order), also as the library's own
    choice, which takes it at the last of these sizes (16 x 2 tiles of 128 rows, 22 x 2 of 96)."""
    def fn(shape):
        def run(a, w, y, *args, **kw):
            ops().gemm_tiled(a, ops().operand_order(w), y, *args, shape=shape, **kw)
        return run
    run_gemm(fn(6), torch.bfloat16, out_dtype, M, N, K)
    a, w = rnd(M, K, dtype=torch.bfloat16, seed=1), ops().operand_order(rnd(N, K, dtype=torch.bfloat16, seed=2))
    ys = []
    for shape in (1, 6, 0):
        y = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops().gemm_tiled(a, w, y, M, N, K, shape=shape)
        ys.append(y)
    assert torch.equal(ys[0], ys[1]) and torch.equal(ys[0], ys[2])
    from spite_amd.csrc.hipops import KernelError
    with pytest.raises(KernelError, match="plain products"):
        ops().gemm_tiled(a[:8, :64].contiguous(), ops().operand_order(rnd(64, 64, dtype=torch.bfloat16)),
                         torch.empty(8, 32, dtype=out_dtype, device=DEV), 8, 32, 64, glu=True, shape=6)


@pytest.mark.parametrize("M,groups", [(40, 150), (300, 150), (9, 64), (70, 65), (500, 129)])
@pytest.mark.parametrize("glu", [False, True])
def test_gemm_over_many_groups(M, groups, glu):
    """More groups than a wave has lanes, most of them empty or with a row or two: the search
    for a row tile's group walks them 64 at a time."""
    N, K = 48, 128
    run_gemm(ops().gemm_generic, torch.float32, torch.float32, M, N, K, glu, True, groups=groups)
    run_gemm(ops().gemm_mfma, torch.bfloat16, torch.float32, M, N, K, glu, True, groups=groups)

    def tiled(a, w, y, *args, **kw):
        ops().gemm_tiled(a, ops().operand_order(w), y, *args, **kw)
    for shape in (1, 3, 4):
        run_gemm(tiled, torch.bfloat16, torch.float32, M, N, K, glu, True, groups=groups, shape=shape)
    if M <= 64:
        # the groups that run_gemm will fill: with the promise that no more hold rows the grid is
        # cut to the row tiles that can exist, and every row must still be served
        cuts = [0] + sorted(torch.randint(0, M + 1, (groups - 1,), generator=torch.Generator().manual_seed(M)).tolist()) + [M]
        live = sum(b > a for a, b in zip(cuts, cuts[1:]))
        assert 0 < live < groups
        for variant in (2, 8, 9):
            def skinny(a, w, y, *args, **kw):
                ops().gemm_skinny(a, ops().operand_order(w), y, *args, tiled=True, variant=variant, **kw)
            run_gemm(skinny, torch.bfloat16, torch.float32, M, N, K, glu, True, groups=groups)
            run_gemm(skinny, torch.bfloat16, torch.float32, M, N, K, glu, True, groups=groups, live_groups=live)
            run_gemm(ops().gemm_skinny, torch.bfloat16, torch.float32, M, N, K, glu, True, groups=groups, variant=variant)


@pytest.mark.parametrize("M,N,K", [(100, 512, 1024), (256, 1040, 2048), (70, 64, 4096), (300, 528, 320), (1, 16, 512)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_tiled_with_the_sum_over_k_cut_into_runs(M, N, K, out_dtype):
    """Few tiles: the wrapper cuts k into runs (also runs of unequal length) and adds them up."""
    from spite_amd.csrc.hipops import tiled_k_runs
    runs = tiled_k_runs(M, N, K)
    assert runs > 1 or K < 512, (M, N, K, runs)
    assert tiled_k_runs(2048, 7168, 5120) == 1          # enough tiles: one run

    def fn(a, w, y, *args, **kw):
        part = torch.empty(runs, M, N, device=DEV) if runs > 1 else None
        ops().gemm_tiled(a, ops().operand_order(w), y, *args, part=part, **kw)
    run_gemm(fn, torch.bfloat16, out_dtype, M, N, K)

    # through the parts' entry, which takes the partial sums from the step's workspace
    from spite_amd.parts.linear import linear, Weight
    from spite_amd.engine.context import Workspace
    a, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    y, ws = torch.empty(M, N, dtype=out_dtype, device=DEV), Workspace(DEV, 1 << 24)
    if M > 64:
        weight = Weight(w)
        linear(a, weight, y, ws=ws)
        assert ws._off >= (runs * M * N * 4 if runs > 1 else 0)    # the partial sums came from the workspace
        ws.reset()
        before = torch.cuda.memory_allocated()
        linear(a, weight, y, ws=ws)
        assert torch.cuda.memory_allocated() == before          # and a warmed-up call allocates nothing
        want = a.float() @ w.float().T
        assert (y.float() - want).abs().max() <= 2e-2 * max(1.0, float(want.abs().max()))


def test_gemm_tiled_refuses_what_it_cannot_do():
    from spite_amd.csrc.hipops import KernelError
    a, w, y = rnd(4, 96, dtype=torch.bfloat16), rnd(32, 96, dtype=torch.bfloat16), rnd(4, 32)
    with pytest.raises(KernelError, match="operand order"):
        ops().gemm_tiled(a, w, y, 4, 32, 96)
    with pytest.raises(KernelError, match="operand order"):
        ops().gemm_skinny(a[:, :72].contiguous(), w[:24, :72].contiguous(), y[:, :24].contiguous(), 4, 24, 72, tiled=True)


def test_gemm_skinny_refuses_what_it_cannot_do():
    from spite_amd.csrc.hipops import KernelError
    a, w, y = rnd(2, 12, dtype=torch.bfloat16), rnd(8, 12, dtype=torch.bfloat16), rnd(2, 8)
    with pytest.raises(KernelError, match="multiples of 8"):
        ops().gemm_skinny(a, w, y, 2, 8, 12)
    with pytest.raises(KernelError, match="bfloat16"):
        ops().gemm_skinny(a.float(), w.float(), y, 2, 8, 12)


# ------------------------------------------------------------------ attention over the paged cache
class PagedKV:
    """Keys and values of a few requests scattered over shuffled pages."""

    def __init__(self, lens, G, hd, ps, dtype, seed=0, extra_pages=3):
        g = torch.Generator().manual_seed(seed)
        self.lens, self.G, self.hd, self.ps = lens, G, hd, ps
        self.k = [torch.randn(n, G, hd, generator=g).to(dtype) for n in lens]
        self.v = [torch.randn(n, G, hd, generator=g).to(dtype) for n in lens]
        blocks = [-(-n // ps) for n in lens]
        n_pages = sum(blocks) + extra_pages
        perm = torch.randperm(n_pages, generator=g).tolist()
        self.tables, at = [], 0
        for b in blocks:
            self.tables.append(perm[at:at + b])
            at += b
        # unused rows hold large values: a kernel that reads beyond a request's keys shows it
        self.kp = torch.full((n_pages, G, ps, hd), 50.0, dtype=dtype)
        self.vp = torch.full((n_pages, G, hd, ps), -70.0, dtype=dtype)
        for s, n in enumerate(lens):
            for j in range(n):
                pg, off = self.tables[s][j // ps], j % ps
                self.kp[pg, :, off] = self.k[s][j]
                self.vp[pg, :, :, off] = self.v[s][j]
        width = max(blocks)
        self.bt = torch.full((len(lens), width), -1, dtype=torch.int32)
        for s, tab in enumerate(self.tables):
            self.bt[s, :len(tab)] = torch.tensor(tab, dtype=torch.int32)

    def drop_below(self, s, first_pos):
        """Gives back the pages wholly below first_pos (their table entries become -1)."""
        for b in range(first_pos // self.ps):
            self.bt[s, b] = -1


def attention_reference(kv, queries, qs, H, vis, span, softcap=0.0, slopes=None):
    """queries: list of (request, position); qs [T,H,hd].  ``slopes`` ([H]): head h's scaled
    score of the key at j gets slopes[h] * (j - p) added; ``softcap``: the scores are then
    capped, softcap * tanh(score / softcap), before the softmax."""
    out = torch.zeros(len(queries), H, kv.hd, dtype=torch.float64)
    for t, (s, p) in enumerate(queries):
        pos = torch.arange(p + 1)
        if p < 8192:
            mask = plain.visible_mask(pos, vis, span)[p:p + 1]
        else:                        # the whole square would not fit: the query's own row of it
            mask = (pos >= plain_first(vis, span, p)).view(1, -1)
        if not softcap and slopes is None:
            out[t] = plain.attention(qs[t:t + 1].double(), kv.k[s][:p + 1].double(), kv.v[s][:p + 1].double(), mask)[0]
            continue
        k, v = kv.k[s][:p + 1].double(), kv.v[s][:p + 1].double()          # [keys, G, hd]
        for h in range(H):
            g = h // (H // k.shape[1])
            score = (k[:, g] @ qs[t, h].double()) / math.sqrt(kv.hd)
            if slopes is not None:
                score = score + float(slopes[h]) * (pos - p).double()
            if softcap:
                score = softcap * torch.tanh(score / softcap)
            score = score.masked_fill(~mask[0], float("-inf"))
            out[t, h] = torch.softmax(score, 0) @ v[:, g]
    return out


def run_attention(kind, dtype, H, G, hd, ps, lens, queries, vis, span, n_splits=3, seed=0, planted=None, softcap=0.0,
                  q_gain=1.0, slopes=None):
    kv = PagedKV(lens, G, hd, ps, dtype, seed)
    T = len(queries)
    g = torch.Generator().manual_seed(seed + 1)
    qs = (torch.randn(T, H, hd, generator=g) * q_gain).to(dtype)
    if planted is not None:                      # one far key that the query must find
        t, s, j = planted
        kv.k[s][j] = (qs[t, ::H // G] * 3.0).to(dtype)
        pg, off = kv.tables[s][j // ps], j % ps
        kv.kp[pg, :, off] = kv.k[s][j]
    for s, first in enumerate([plain_first(vis, span, max([p for ss, p in queries if ss == s], default=0))
                               for s in range(len(lens))]):
        low = min([plain_first(vis, span, p) for ss, p in queries if ss == s], default=0)
        kv.drop_below(s, low)
    ref = attention_reference(kv, queries, qs, H, vis, span, softcap, slopes)
    sl = None if slopes is None else torch.tensor(slopes, dtype=torch.float32, device=DEV)
    positions = torch.tensor([p for _, p in queries], dtype=torch.int32, device=DEV)
    seq = torch.tensor([s for s, _ in queries], dtype=torch.int32, device=DEV)
    out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
    q_dev, kp, vp, bt = qs.reshape(T, H * hd).to(DEV), kv.kp.to(DEV), kv.vp.to(DEV), kv.bt.to(DEV)
    scale = 1.0 / math.sqrt(hd)
    if kind != "generic":                        # the MFMA kernels read pages in operand order
        kp, vp = ops().kv_operand_order(kp, vp)
    if kind == "generic":
        ops().attn_generic(q_dev, kp, vp, out, positions, seq, bt, T, H, G, hd, ps, vis, span, scale, softcap=softcap, slopes=sl)
        if ops().kv_tiled_ok(dtype, hd, ps):     # and the plain kernel reads them too, with the same bits
            again = torch.zeros_like(out)
            kpt, vpt = ops().kv_operand_order(kp, vp)
            ops().attn_generic(q_dev, kpt, vpt, again, positions, seq, bt, T, H, G, hd, ps, vis, span, scale, kv_tiled=True,
                               softcap=softcap, slopes=sl)
            assert torch.equal(out, again)
    elif kind == "prefill":                      # runs of queries of one request are the portions
        runs = []
        for s, _ in queries:
            if runs and runs[-1][0] == s:
                runs[-1][1] += 1
            else:
                runs.append([s, 1])
        cu = torch.tensor([0] + list(np.cumsum([c for _, c in runs])), dtype=torch.int32, device=DEV)
        ops().attn_prefill(q_dev, kp, vp, out, positions, cu, [c for _, c in runs],
                           bt[[s for s, _ in runs]].contiguous(), H, G, hd, ps, vis, span, scale, softcap=softcap, slopes=sl)
    else:
        wsz = ops().attn_decode_workspace(T, H, hd, n_splits)
        scratch = torch.empty(wsz // 4, dtype=torch.float32, device=DEV)
        ops().attn_decode(q_dev, kp, vp, out, scratch, positions, seq, bt, T, H, G, hd, ps, vis, span, scale, n_splits,
                          softcap=softcap, slopes=sl)
    got = out.double().cpu().view(T, H, hd)
    err = (got - ref).abs().max()
    assert torch.isfinite(got).all()
    # bf16: P is rounded as an MFMA operand and the output once
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    assert err < tol * max(1.0, float(ref.abs().max())), err
    return got, ref


def plain_first(vis, span, p):
    return {"full": 0, "chunk": (p // span) * span if span else 0, "window": max(p - span + 1, 0) if span else 0}[vis]


ATT_CASES = [
    # H, G, hd, page, lens, queries (request, position), visibility, span
    (4, 2, 16, 4, [9, 30], [(0, 8), (1, 29), (1, 3), (0, 0)], "full", 0),
    (6, 3, 24, 8, [70], [(0, 69), (0, 16), (0, 15), (0, 32)], "chunk", 16),
    (6, 3, 24, 8, [70], [(0, 69), (0, 20), (0, 19), (0, 5)], "window", 20),
    (5, 1, 64, 32, [200, 64], [(0, 199), (1, 63), (0, 64), (0, 31), (0, 32)], "full", 0),
    (8, 2, 128, 64, [300], [(0, 299), (0, 255), (0, 256), (0, 128)], "chunk", 128),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATT_CASES, ids=lambda c: f"H{c[0]}G{c[1]}hd{c[2]}ps{c[3]}{c[6]}")
def test_attn_generic(dtype, case):
    H, G, hd, ps, lens, queries, vis, span = case
    run_attention("generic", dtype, H, G, hd, ps, lens, queries, vis, span)


DEC_CASES = [
    (5, 1, 64, 32, [200, 64, 1], [(0, 199), (1, 63), (2, 0)], "full", 0),
    (8, 2, 128, 64, [300, 129], [(0, 299), (1, 128)], "chunk", 128),
    (40, 8, 128, 64, [1000, 33, 4096], [(0, 999), (1, 32), (2, 4095)], "full", 0),
    (16, 1, 64, 32, [500], [(0, 499)], "window", 100),
    (12, 4, 128, 32, [260, 70], [(0, 259), (1, 69)], "chunk", 64),
]


@pytest.mark.parametrize("n_splits", [1, 3, 16])
@pytest.mark.parametrize("case", DEC_CASES, ids=lambda c: f"H{c[0]}G{c[1]}hd{c[2]}ps{c[3]}{c[6]}")
def test_attn_decode(case, n_splits):
    H, G, hd, ps, lens, queries, vis, span = case
    run_attention("decode", torch.bfloat16, H, G, hd, ps, lens, queries, vis, span, n_splits)


PORTION_CASES = [
    # H, G, hd, page, cached lengths after the step, portions (request, first position, count), visibility, span
    (5, 1, 64, 32, [200, 70, 1], [(0, 120, 80), (1, 0, 70), (2, 0, 1)], "full", 0),
    (8, 2, 128, 64, [300], [(0, 0, 300)], "chunk", 128),
    (8, 2, 128, 64, [300, 40], [(0, 250, 50), (1, 39, 1)], "chunk", 128),       # a portion across a chunk border
    (40, 8, 128, 64, [130, 65], [(0, 97, 33), (1, 0, 65)], "full", 0),
    (16, 1, 64, 32, [500], [(0, 380, 120)], "window", 100),
    (12, 4, 128, 32, [260, 70], [(0, 258, 2), (1, 0, 70)], "chunk", 64),
    (6, 2, 128, 64, [900], [(0, 0, 900)], "full", 0),                          # 3 heads a kv head: tiles of 85 queries
    (2, 2, 64, 32, [600, 3], [(0, 100, 500), (1, 0, 3)], "full", 0),           # one head a kv head: tiles of 256
    (40, 8, 128, 64, [700], [(0, 300, 400)], "window", 257),
    (34, 2, 64, 96, [400], [(0, 0, 400)], "full", 0),                          # 17 heads a kv head, pages of 96
    (40, 1, 64, 32, [333, 9], [(0, 280, 53), (1, 0, 9)], "chunk", 160),          # 40 heads a kv head: a wave's columns are one query's
    # the first visible key (96) lies on a page with an odd index: the block of 64 keys that holds it
    # begins on a page that was given back
    (16, 1, 64, 32, [500], [(0, 195, 120)], "window", 100),
    (10, 2, 128, 32, [400, 50], [(0, 230, 90), (1, 10, 40)], "chunk", 96),
]


@pytest.mark.parametrize("n_splits", [1, 2, 5])
@pytest.mark.parametrize("case", PORTION_CASES, ids=lambda c: f"H{c[0]}G{c[1]}hd{c[2]}ps{c[3]}{c[6]}")
def test_attn_prefill(case, n_splits):
    H, G, hd, ps, lens, portions, vis, span = case
    dtype = torch.bfloat16
    kv = PagedKV(lens, G, hd, ps, dtype, seed=3)
    queries = [(s, p) for s, first, count in portions for p in range(first, first + count)]
    T = len(queries)
    g = torch.Generator().manual_seed(4)
    qs = torch.randn(T, H, hd, generator=g).to(dtype)
    for s, first, count in portions:
        kv.drop_below(s, plain_first(vis, span, first))
    # pages that no request holds (given back, or never handed out) are somebody else's: nothing of
    # them may reach the output, not even through a probability of zero
    held = {int(p) for p in kv.bt.flatten().tolist() if p >= 0}
    for p in range(kv.kp.shape[0]):
        if p not in held:
            kv.kp[p], kv.vp[p] = float("nan"), float("nan")
    ref = attention_reference(kv, queries, qs, H, vis, span)
    positions = torch.tensor([p for _, p in queries], dtype=torch.int32, device=DEV)
    seq = torch.tensor([i for i, (s, first, count) in enumerate(portions) for _ in range(count)], dtype=torch.int32, device=DEV)
    cu = [0]
    for _, _, count in portions:
        cu.append(cu[-1] + count)
    bt = torch.stack([kv.bt[s] for s, _, _ in portions]).to(DEV)
    out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
    ops().attn_prefill(qs.reshape(T, H * hd).to(DEV), *ops().kv_operand_order(kv.kp.to(DEV), kv.vp.to(DEV)), out, positions,
                       torch.tensor(cu, dtype=torch.int32, device=DEV), [count for _, _, count in portions], bt,
                       H, G, hd, ps, vis, span, 1.0 / math.sqrt(hd), n_splits=n_splits,
                       scratch=torch.full((ops().attn_prefill_workspace([c for _, _, c in portions], H, G, hd, n_splits) // 4 + 1,),
                                          float("nan"), device=DEV))
    got = out.double().cpu().view(T, H, hd)
    assert torch.isfinite(got).all()
    assert (got - ref).abs().max() < 1.5e-2 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("kind,dtype", [("generic", torch.float32), ("generic", torch.bfloat16), ("decode", torch.bfloat16),
                                        ("prefill", torch.bfloat16)])
def test_attention_with_capped_scores(kind, dtype):
    """Scores capped smoothly before the softmax (an option of every attention kernel): queries
    three times as long as usual, so that scores reach beyond the cap of 4 and the cap matters."""
    H, G, hd, ps = (8, 2, 128, 64) if kind != "generic" else (6, 3, 24, 8)
    queries = [(0, p) for p in range(250, 300)] if kind == "prefill" else [(0, 299), (1, 128), (0, 40)]
    if kind == "prefill":
        queries += [(1, p) for p in range(0, 129)]
    else:
        queries = sorted(queries)
    got, ref = run_attention(kind, dtype, H, G, hd, ps, [300, 129], queries, "chunk", 128, softcap=4.0, q_gain=3.0)
    # without the cap the result is another one
    kv = PagedKV([300, 129], G, hd, ps, dtype, 0)
    g = torch.Generator().manual_seed(1)
    qs = (torch.randn(len(queries), H, hd, generator=g) * 3.0).to(dtype)
    other = attention_reference(kv, queries, qs, H, "chunk", 128)
    assert (other - ref).abs().max() > 0.1


@pytest.mark.parametrize("softcap", [0.0, 3.0])
@pytest.mark.parametrize("kind,dtype", [("generic", torch.float32), ("generic", torch.bfloat16), ("decode", torch.bfloat16),
                                        ("prefill", torch.bfloat16)])
def test_attention_with_score_slopes(kind, dtype, softcap):
    """A bias slope * (key - query position) per head on the scaled scores (an option of every
    attention kernel), alone and before a cap: steep on some heads (they read their last few
    keys), flat on others, zero on one."""
    H, G, hd, ps = (8, 2, 128, 64) if kind != "generic" else (6, 3, 24, 8)
    slopes = [0.0, 0.004, 0.03, 0.25, 1.0, 0.5, 0.06, 0.008][:H]
    queries = [(0, p) for p in range(230, 300)] if kind == "prefill" else [(0, 299), (1, 128), (0, 40)]
    if kind == "prefill":
        queries += [(1, p) for p in range(0, 129)]
    else:
        queries = sorted(queries)
    got, ref = run_attention(kind, dtype, H, G, hd, ps, [300, 129], queries, "full", 0, softcap=softcap, slopes=slopes)
    kv = PagedKV([300, 129], G, hd, ps, dtype, 0)
    g = torch.Generator().manual_seed(1)
    qs = torch.randn(len(queries), H, hd, generator=g).to(dtype)
    other = attention_reference(kv, queries, qs, H, "full", 0, softcap)
    assert (other[:, 1:] - ref[:, 1:]).abs().max() > 0.1          # the slopes matter ...
    assert (other[:, 0] - ref[:, 0]).abs().max() < 1e-12          # ... and a slope of zero changes nothing


def test_prefill_attention_finds_one_far_key_among_thousands():
    # as below, for one query in the middle of a portion of 100: the far key lies in a block
    # that every query of the tile sees whole
    queries = [(0, p) for p in range(2900, 3000)]
    got, ref = run_attention("prefill", torch.bfloat16, 8, 2, 128, 64, [3000], queries, "full", 0, planted=(50, 0, 77))
    kv = PagedKV([3000], 2, 128, 64, torch.bfloat16, 0)
    assert (ref[50, 0] - kv.v[0][77][0].double()).abs().max() < 0.05
    assert (got - ref).abs().max() < 2e-2


@pytest.mark.parametrize("kind", ["generic", "decode"])
def test_attention_finds_one_far_key_among_thousands(kind):
    # random keys give nearly uniform weights, which would hide a key that is skipped: one key
    # far back matches the query, and the output must be close to that key's value
    got, ref = run_attention(kind, torch.bfloat16, 8, 2, 128, 64, [3000], [(0, 2999)], "full", 0, n_splits=7,
                             planted=(0, 0, 77))
    # the reference itself puts nearly all the weight on key 77: its output is that key's value
    kv = PagedKV([3000], 2, 128, 64, torch.bfloat16, 0)
    assert (ref[0, 0] - kv.v[0][77][0].double()).abs().max() < 0.05
    assert (got - ref).abs().max() < 2e-2


@pytest.mark.parametrize("kind,vis,span,far,n_splits", [
    ("decode", "full", 0, 123, 64), ("decode", "full", 0, 20000, 256), ("decode", "chunk", 8192, 32768, 16),
    ("prefill", "full", 0, 123, 0), ("prefill", "chunk", 8192, 32769, 0)])
def test_attention_at_forty_thousand_keys(kind, vis, span, far, n_splits):
    """Positions beyond the real model's first chunk borders, page tables of hundreds of pages: one
    far key (the first ones of the context, or of the query's chunk) carries the answer."""
    n = 40000
    queries = [(0, n - 1)] if kind == "decode" else [(0, p) for p in range(n - 18, n)]
    t = len(queries) // 2
    got, ref = run_attention(kind, torch.bfloat16, 4, 1, 128, 64, [n], queries, vis, span, n_splits=n_splits, planted=(t, 0, far))
    kv = PagedKV([n], 1, 128, 64, torch.bfloat16, 0)
    assert (ref[t, 0] - kv.v[0][far][0].double()).abs().max() < 0.05
    assert (got - ref).abs().max() < 2e-2


@pytest.mark.parametrize("kind", ["generic", "decode"])
def test_attention_refuses_what_it_cannot_do(kind):
    from spite_amd.csrc.hipops import KernelError
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    i32 = lambda *s: torch.zeros(*s, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError):
        if kind == "generic":
            ops().attn_generic(z(1, 6 * 16), z(1, 4, 8, 16), z(1, 4, 16, 8), z(1, 6 * 16), i32(1), i32(1), i32(1, 4),
                               1, 6, 4, 16, 8, "full", 0, 0.25)        # 6 heads over 4 kv heads
        else:
            ops().attn_decode(z(1, 4 * 48), z(1, 2, 32, 48), z(1, 2, 48, 32), z(1, 4 * 48),
                              torch.zeros(4096, device=DEV), i32(1), i32(1), i32(1, 4), 1, 4, 2, 48, 32, "full", 0,
                              0.1, 1)                                    # head size 48


# ------------------------------------------------------------------ router, expert plan, sampling
@pytest.mark.parametrize("T,d,E", [(1, 64, 4), (9, 5120, 16), (300, 96, 8), (70, 1002, 128), (1029, 520, 16)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_with_projection_and_plan_from_logits_match_the_router(T, d, E, out_dtype):
    # the norm forms the router's logits in its own pass and the plan kernel takes the choice from
    # them: the same bits as the three kernels in a row give
    h = rnd(T, d, seed=5)
    delta = rnd(T, d, seed=6)
    w, wr = rnd(d, seed=7) + 1.0, rnd(E, d, seed=8)
    wr[3 % E] = wr[1 % E]
    out_a, out_b = torch.empty(T, d, dtype=out_dtype, device=DEV), torch.empty(T, d, dtype=out_dtype, device=DEV)
    x32 = torch.empty(T, d, device=DEV)
    h_a, h_b = h.clone(), h.clone()
    ops().add_rmsnorm(h_a, w, 1e-5, out=out_a, out32=x32, d1=delta)
    expert_a = torch.empty(T, dtype=torch.int32, device=DEV)
    weight_a = torch.empty(T, device=DEV)
    logits_a = torch.empty(T, E, device=DEV)
    ops().router_top1(x32, wr, expert_a, weight_a, logits_a)
    logits_b = torch.empty(T, E, device=DEV)
    ops().add_rmsnorm(h_b, w, 1e-5, out=out_b, d1=delta, proj=wr, proj_out=logits_b)
    assert torch.equal(h_a, h_b) and torch.equal(out_a, out_b) and torch.equal(logits_a, logits_b)
    n = 2 * T
    plans = []
    for logits in (None, logits_b):
        expert = expert_a.clone() if logits is None else torch.full((T,), -7, dtype=torch.int32, device=DEV)
        weight = weight_a.clone() if logits is None else torch.zeros(T, device=DEV)
        src, dst = torch.empty(n, dtype=torch.int32, device=DEV), torch.empty(n, dtype=torch.int32, device=DEV)
        scale, offsets = torch.empty(n, device=DEV), torch.empty(E + 2, dtype=torch.int32, device=DEV)
        ops().moe_plan(expert, weight, src, scale, dst, offsets, T, E, True, logits=logits)
        plans.append((expert, weight, src, dst, scale, offsets))
    for a, b in zip(*plans):
        assert torch.equal(a, b)


def test_router_bits_do_not_depend_on_how_many_tokens_a_step_brings():
    T, d, E = 1029, 520, 16                                 # many tokens share a workgroup; fewer than 256 do not
    x, wr = rnd(T, d), rnd(E, d, seed=2)
    out = {}
    for name, rows in (("all", [(0, T)]), ("pieces", [(0, 200), (200, 455), (455, 456), (456, T)])):
        expert = torch.empty(T, dtype=torch.int32, device=DEV)
        weight = torch.empty(T, dtype=torch.float32, device=DEV)
        logits = torch.empty(T, E, dtype=torch.float32, device=DEV)
        for b, e in rows:
            ops().router_top1(x[b:e], wr, expert[b:e], weight[b:e], logits[b:e])
        out[name] = (expert.cpu(), weight.cpu(), logits.cpu())
    for a, b in zip(out["all"], out["pieces"]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("T,d,E", [(1, 64, 4), (9, 96, 8), (70, 5120, 16), (33, 1000, 128), (300, 512, 16), (1029, 96, 8),
                                   (2050, 64, 300)])
def test_router_and_plan(T, d, E):
    x = rnd(T, d)
    wr = rnd(E, d, seed=2)
    wr[3 % E] = wr[1 % E]                                   # two experts with equal logits: the lower index wins
    expert = torch.empty(T, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, dtype=torch.float32, device=DEV)
    logits = torch.empty(T, E, dtype=torch.float32, device=DEV)
    ops().router_top1(x, wr, expert, weight, logits)
    idx, w, lg = plain.router_top1(x.double().cpu(), wr.double().cpu())
    assert (logits.double().cpu() - lg).abs().max() < 2e-5 * lg.abs().max()
    # where the plain side's two best logits are not within rounding of each other, the choice is the same
    top2 = torch.topk(lg, 2, dim=-1).values
    sure = (top2[:, 0] - top2[:, 1]) > 1e-4 * lg.abs().max()
    assert torch.equal(expert.cpu().long()[sure], idx[sure])
    assert not (expert.cpu() == 3 % E).any() or E <= 3      # the duplicate with the higher index is never taken
    if sure.any():
        assert (weight.double().cpu()[sure] - w[sure]).abs().max() < 1e-5
    n = 2 * T
    src, dst = torch.empty(n, dtype=torch.int32, device=DEV), torch.empty(n, dtype=torch.int32, device=DEV)
    scale = torch.empty(n, dtype=torch.float32, device=DEV)
    offsets = torch.empty(E + 2, dtype=torch.int32, device=DEV)
    ops().moe_plan(expert, weight, src, scale, dst, offsets, T, E, True)
    e, off, s_, d_ = expert.cpu().tolist(), offsets.cpu().tolist(), src.cpu().tolist(), dst.cpu().tolist()
    assert off[0] == 0 and off[E] == T and off[E + 1] == 2 * T
    for g in range(E):
        members = s_[off[g]:off[g + 1]]
        assert members == [t for t in range(T) if e[t] == g]        # stable: tokens in order inside a group
    assert s_[T:] == list(range(T)) and d_[:T] == s_[:T] and d_[T:] == list(range(T, 2 * T))
    assert torch.equal(scale[:T].cpu(), weight.cpu()[torch.tensor(s_[:T])]) and (scale[T:] == 1).all()


@pytest.mark.parametrize("V", [7, 384, 202048])
def test_argmax_and_sampling_rows(V):
    from spite_amd.sampling.sampler import lcg_next
    n = 5
    logits = rnd(n, V, scale=3.0)
    logits[0, V // 2] = logits[0].max() + 1
    logits[1, 1] = logits[1, V - 2] = logits[1].max() + 2                  # a tie: the first wins
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    sv, si = torch.empty(32 * n, device=DEV), torch.empty(32 * n, dtype=torch.int32, device=DEV)
    ops().argmax_rows(logits, out, sv, si)
    want = [plain.greedy(r) for r in logits.cpu()]
    assert out.cpu().tolist() == want and want[0] == V // 2 and want[1] == 1
    ops().sample_rows(logits, None, None, out)
    assert out.cpu().tolist() == want
    # draws: the same uniform numbers as the plain sampler's generator gives
    temps = torch.tensor([0.0, 0.7, 1.0, 1.3, 2.0], device=DEV)
    states, us, plain_tokens = [11, 12, 13, 14, 15], [], []
    for r in range(n):
        if float(temps[r]) > 0:
            t, _ = plain.multinomial(logits[r].cpu() / float(temps[r]), states[r])
            _, u = lcg_next(states[r])
        else:
            t, u = want[r], 0.0
        plain_tokens.append(t)
        us.append(u)
    ops().sample_rows(logits, temps, torch.tensor(us, device=DEV), out)
    got = out.cpu().tolist()
    for r in range(n):
        if got[r] != plain_tokens[r]:
            # Both walk a float32 running sum over V terms, in different groupings; the sums
            # differ by about sqrt(V) * 2^-24 of the total, so the two indices may lie apart
            # by that much probability mass (and both must sit at the drawn number)
            p = torch.softmax(logits[r].double().cpu() / float(temps[r]), 0)
            cdf = torch.cumsum(p, 0)
            slack = 4 * math.sqrt(V) * 2.0 ** -24 + 1e-6
            assert abs(float(cdf[got[r]] - cdf[plain_tokens[r]])) < slack, (r, got[r], plain_tokens[r])
            assert abs(float(cdf[got[r]]) - us[r]) < slack + float(p[got[r]])
    # rows that were filtered to -inf are never drawn
    masked = logits.clone()
    masked[:, 1:] = float("-inf")
    ops().sample_rows(masked, torch.ones(n, device=DEV), torch.rand(n, device=DEV), out)
    assert out.cpu().tolist() == [0] * n


def _filter_case(row, ctx, temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, penalty=1.0, last_n=0):
    l = plain.apply_repetition_penalty(row.clone(), ctx, penalty, last_n)
    l = plain.apply_temperature(l, temperature)
    l = plain.apply_min_p(l, min_p)
    l = plain.apply_top_k(l, top_k)
    return plain.apply_top_p(l, top_p)


@pytest.mark.parametrize("V", [7, 1000, 20011])
def test_filter_rows_against_the_plain_filters(V):
    """Every filter alone, all together, a row left alone, ties at both thresholds."""
    from spite_amd.sampling.sampler import Sampler, SamplingParams
    g = torch.Generator().manual_seed(V)
    cases = [dict(), dict(temperature=0.7), dict(top_k=3, temperature=1.0), dict(top_p=0.6, temperature=1.3),
             dict(min_p=0.2, temperature=1.0), dict(penalty=1.4, last_n=0), dict(penalty=1.3, last_n=2, temperature=0.9),
             dict(temperature=0.8, top_k=min(50, V - 1), top_p=0.9, min_p=0.01, penalty=1.2, last_n=0),
             dict(top_k=4, temperature=1.0), dict(top_p=0.5, temperature=1.0),
             dict(min_p=0.3, top_k=40, temperature=1.0), dict(top_k=5, temperature=1.0),
             dict(top_p=0.999, temperature=1.0), dict(top_p=0.9, temperature=1.0), dict(top_k=300, temperature=1.0),
             dict(top_k=37, top_p=0.5, temperature=1.0)]
    n = len(cases)
    logits = torch.randn(n, V, generator=g) * 3.0
    # ties: rows 8 and 9 hold few distinct values, so that the k-th largest and the value at
    # which the mass reaches p are shared by several elements (with a large vocabulary by more
    # than the kernel sorts in one go: its digit-by-digit search runs)
    few = 2 if V > 20000 else 4
    logits[8] = torch.randint(0, few, (V,), generator=g).float()
    logits[9] = torch.randint(0, few - 1 if few > 2 else 2, (V,), generator=g).float() * 0.5
    # row 10: min-p leaves fewer values than top-k asks for.  Row 11: three values far above
    # the rest, so that the fifth largest lies in the far tail.  Row 12: nearly all the mass.
    logits[11, [1, V // 2, V - 1]] += 100.0
    # rows 13 to 15: nearly flat (what random weights give): one bin of the kernel's first look
    # holds everything, its finer bins have to tell the elements apart
    logits[13:16] *= 0.004
    ctxs = [[int(x) for x in torch.randint(0, V, (9,), generator=g)] + [V + 5, -1] for _ in range(n)]
    params = [SamplingParams(temperature=c.get("temperature", 0.0), top_k=c.get("top_k", 0), top_p=c.get("top_p", 1.0),
                             min_p=c.get("min_p", 0.0), repetition_penalty=c.get("penalty", 1.0),
                             repeat_last_n=c.get("last_n", 64)) for c in cases]
    work = logits.to(DEV).clone()
    Sampler(DEV)._filter(work, params, ctxs)
    got = work.cpu()
    for r, c in enumerate(cases):
        if not params[r].filters():
            assert torch.equal(got[r], logits[r]), r          # rows that ask for nothing are not touched
            continue
        want = _filter_case(logits[r], [t for t in ctxs[r]], **c)
        assert torch.equal(torch.isinf(got[r]), torch.isinf(want)), (r, c, int(torch.isinf(got[r]).sum()), int(torch.isinf(want).sum()))
        keep = ~torch.isinf(want)
        assert torch.equal(got[r][keep], want[keep]), (r, c)
    # top-k keeps every element equal to the k-th largest; top-p the first of the equal ones
    kept8 = (~torch.isinf(got[8])).nonzero().flatten()
    assert len(kept8) >= 4
    if int((logits[8] == logits[8].max()).sum()) >= 4:
        assert bool((logits[8][kept8] == logits[8].max()).all())
    kept9 = (~torch.isinf(got[9])).nonzero().flatten().tolist()
    top = (logits[9] == logits[9].max()).nonzero().flatten().tolist()
    assert kept9 == top[:len(kept9)] or set(top) <= set(kept9)


def test_randn_fill_is_normal_and_depends_on_seed_key_and_index_alone():
    n = 1 << 20
    a = torch.empty(n, device=DEV)
    ops().randn_fill(a, 7, 99, 0.0, 1.0)
    assert abs(float(a.mean())) < 5e-3 and abs(float(a.std()) - 1.0) < 5e-3
    z = a.double().cpu()
    # the shape of the distribution: its fourth moment, and the share beyond two deviations
    assert abs(float((z ** 4).mean()) - 3.0) < 0.1 and abs(float((z.abs() > 2).double().mean()) - 0.0455) < 2e-3
    # neighbours (the two normals of one pair, and those of adjacent pairs) are uncorrelated
    for lag in (1, 2, 3):
        assert abs(float((z[:-lag] * z[lag:]).mean())) < 5e-3
    # the same call gives the same numbers; a longer tensor starts with them; mean and deviation scale them
    b = torch.empty(n + 5, device=DEV)
    ops().randn_fill(b, 7, 99, 1.0, 0.02)
    assert torch.allclose(b[:n], 1.0 + 0.02 * a, atol=1e-6)
    c = torch.empty(n, device=DEV)
    ops().randn_fill(c, 7, 99, 0.0, 1.0)
    assert torch.equal(a, c)
    # another key or another seed: other numbers
    for seed, key in ((7, 100), (8, 99)):
        ops().randn_fill(c, seed, key, 0.0, 1.0)
        assert abs(float((a * c).mean())) < 5e-3 and not torch.equal(a, c)
    # bfloat16 holds the rounded values; an odd length fills its last element
    h = torch.empty(1001, dtype=torch.bfloat16, device=DEV)
    ops().randn_fill(h, 7, 99, 0.0, 1.0)
    assert torch.equal(h, a[:1001].to(torch.bfloat16))


def test_randn_fill_equals_its_host_port_bit_for_bit():
    # the folder writer draws on the host what the engine's random-weights mode draws on the GPU
    import numpy as np
    from spite_amd.weights.random_init import normal_numbers
    n = (1 << 20) + 1
    for seed, key, mean, std in ((7, 99, 0.0, 1.0), (123456789012345, 0xfedcba98, 1.0, 0.02), (0, 0, 0.0, 0.05)):
        host = normal_numbers(n, seed, key, mean, std)
        a = torch.empty(n, device=DEV)
        ops().randn_fill(a, seed, key, mean, std)
        assert np.array_equal(a.cpu().numpy().view(np.uint32), host.view(np.uint32)), (seed, key)
        h = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        ops().randn_fill(h, seed, key, mean, std)
        assert torch.equal(h.cpu(), torch.from_numpy(host).to(torch.bfloat16))


def test_mfma_loop_runs_and_counts_its_flops():
    """The benchmark's loop of MFMAs alone: it finishes, writes a sum per workgroup, and on zero
    operands every sum is zero."""
    out = torch.full((8,), -1.0, device=DEV)
    flops = ops().mfma_loop(out, 10, 0.0)
    torch.cuda.synchronize()
    assert flops == 8 * 8 * 10 * 32 * 16384 and float(out.abs().sum()) == 0.0
    # the sums are the loop's work: twice the steps give twice the sums (the same products are
    # added again), operands of half the size a quarter (exactly: a power of two); a loop that
    # dropped or repeated products would break the first, one that ignored its operands the second
    def sums(steps, gain):
        ops().mfma_loop(out, steps, gain)
        torch.cuda.synchronize()
        return out.double().cpu()
    one, two, half = sums(10, 1.0), sums(20, 1.0), sums(10, 0.5)
    assert torch.isfinite(one).all() and float(one.abs().max()) > 0.0 and one.unique().numel() > 1
    assert float((two - 2 * one).abs().max()) <= 1e-4 * float(one.abs().max())
    assert torch.equal(half * 4, one)
