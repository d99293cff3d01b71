"""Plain, slow Llama 4 text model: whole sequences, no cache, one function per part.

Written from the formulas of giveen/spite (cited per function as path:line under the
reference checkout) and shares no code with ``spite_amd``.  Everything runs on the CPU in
float64 unless a dtype is given.  The only inputs are a plain ``dict`` of hyper-parameters
(the keys of a Llama 4 ``config.json``) and a ``dict`` name -> tensor in the on-disk
layout (``[out, in]`` matrices; experts ``gate_up_proj [E, d, 2F]``, ``down_proj [E, F, d]``).
"""
from __future__ import annotations

import math

import torch

# --------------------------------------------------------------------------- norms


def rms_norm(x: torch.Tensor, w: torch.Tensor | None, eps: float) -> torch.Tensor:
    """crates/spite-models/src/dense.rs:175-181: ms = sum(x^2)/n; y = x * 1/sqrt(ms+eps) * w."""
    ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    y = x * (1.0 / torch.sqrt(ms + eps))
    return y if w is None else y * w


def qk_l2_norm(x: torch.Tensor, eps: float) -> torch.Tensor:
    """crates/spite-models/src/llama/llama4.rs:160-175: per head, rmsnorm with a weight of
    ones, after the rotation.  ``x`` is ``[T, heads, hd]``."""
    return rms_norm(x, None, eps)


# --------------------------------------------------------------------------- position encoding


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """crates/spite-rope/src/lib.rs:81: f_i = 1 / theta^(2i/hd), i < hd/2.

    The reference has no frequency scaling (llama4.rs:97-101 passes RopeVariant::Default);
    the ``llama3`` rule is the one named by the configuration key ``rope_scaling``:
    wavelength L = 2*pi/f; L < orig/high -> f; L > orig/low -> f/factor; between, a linear
    blend with s = (orig/L - low)/(high - low): (1-s)*f/factor + s*f.
    """
    half = head_dim // 2
    i = torch.arange(half, dtype=torch.float64)
    f = 1.0 / (float(theta) ** (2.0 * i / head_dim))
    if scaling is None:
        return f
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind != "llama3":
        raise ValueError(f"plain implementation knows rope_type llama3 only, got {kind!r}")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    out = []
    for fi in f.tolist():
        wavelen = 2.0 * math.pi / fi
        if wavelen < orig / high:
            out.append(fi)
        elif wavelen > orig / low:
            out.append(fi / factor)
        else:
            s = (orig / wavelen - low) / (high - low)
            out.append((1.0 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=torch.float64)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
               pairing: str = "half", angle_dtype=None) -> torch.Tensor:
    """crates/spite-rope/src/lib.rs:78-92 (rope_range): half-split pairs (i, i+hd/2):
    x_i' = x_i cos a - x_{i+half} sin a ; x_{i+half}' = x_i sin a + x_{i+half} cos a,
    a = pos * f_i; every head alike (lib.rs:69-71).  ``x`` is ``[T, heads, hd]``.
    ``pairing="adjacent"`` pairs (2i, 2i+1) instead (not the reference's).
    ``angle_dtype=torch.float32``: position, frequency and their product in 32-bit, as
    lib.rs:82 forms them (``pos as f32 * freq``): at position p that angle is off by up to
    p * 2^-24 rad, a thousandth at 17,000; sine and cosine of the rounded angle are then exact
    here.  Default: everything in the dtype of ``x``."""
    hd = x.shape[-1]
    half = hd // 2
    adt = angle_dtype or x.dtype
    ang = (positions.to(adt)[:, None] * inv_freq.to(adt)[None, :]).to(x.dtype)  # [T, half]
    cos = torch.cos(ang)[:, None, :]
    sin = torch.sin(ang)[:, None, :]
    out = torch.empty_like(x)
    if pairing == "half":
        x0, x1 = x[..., :half], x[..., half:]
        out[..., :half] = x0 * cos - x1 * sin
        out[..., half:] = x0 * sin + x1 * cos
    elif pairing == "adjacent":
        x0, x1 = x[..., 0::2], x[..., 1::2]
        out[..., 0::2] = x0 * cos - x1 * sin
        out[..., 1::2] = x0 * sin + x1 * cos
    else:
        raise ValueError(pairing)
    return out


def attn_temperature(positions: torch.Tensor, floor_scale: int, attn_scale: float,
                     dtype=torch.float64) -> torch.Tensor:
    """crates/spite-models/src/llama/llama4.rs:178-183:
    scale = ln(floor((pos+1)/S) + 1) * alpha + 1 with integer division (S=8192, alpha=0.1
    fixed there; configuration keys ``floor_scale`` / ``attn_scale`` here)."""
    k = torch.div(positions.to(torch.int64) + 1, int(floor_scale), rounding_mode="floor")
    return torch.log(k.to(dtype) + 1.0) * attn_scale + 1.0


# --------------------------------------------------------------------------- attention


def visible_mask(positions: torch.Tensor, kind: str, size: int = 0, key_positions=None) -> torch.Tensor:
    """``mask[p, j]`` true when the query at position p may read the key at position j
    (``key_positions``: the keys' positions when they are not the queries' own).

    * ``full``: causal, j <= p (crates/spite-compute/src/flash_attn.rs:118-121).
    * ``window``: causal and among the last ``size`` rows, j > p - size
      (crates/spite-models/src/llama/llama4.rs:189-197, what the reference computes).
    * ``chunk``: causal and floor(j/size) == floor(p/size): the chunked attention that the
      configuration key ``attention_chunk_size`` names (the reference's comments call its
      window "chunked", llama4.rs:6, but compute no chunks).
    """
    p = positions.to(torch.int64)[:, None]
    j = (positions if key_positions is None else key_positions).to(torch.int64)[None, :]
    m = j <= p
    if kind == "full":
        return m
    if kind == "window":
        return m & (j > p - size)
    if kind == "chunk":
        return m & (torch.div(j, size, rounding_mode="floor") == torch.div(p, size, rounding_mode="floor"))
    raise ValueError(kind)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """crates/spite-compute/src/flash_attn.rs:71-158.  q ``[T,H,hd]``, k/v ``[S,G,hd]``,
    mask ``[T,S]``.  Head h reads kv head h // (H/G) (:89,114); score = (q.k) / sqrt(hd)
    (:57,124-125); softmax with the row maximum subtracted, sum floored at 1e-30 (:129-143);
    o = sum_j p_j v_j (:146-154)."""
    T, H, hd = q.shape
    G = k.shape[1]
    rep = H // G
    scale = 1.0 / math.sqrt(hd)
    out = torch.zeros_like(q)
    for h in range(H):
        g = h // rep
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        p = torch.exp(s - m)
        z = p.sum(-1, keepdim=True).clamp_min(1e-30)
        out[:, h, :] = (p / z) @ v[:, g, :]
    return out


def attention_rows(q, k, v, q_pos, kind: str, size: int = 0, key_start: int = 0, block: int = 1024) -> torch.Tensor:
    """``attention`` for queries at positions ``q_pos`` (ascending) over keys at positions
    ``key_start`` .. ``key_start + S - 1``, a block of queries at a time, so that a long
    sequence never needs its whole score matrix at once.  A block only meets the keys from the
    first one that its first query may read to its last query's own."""
    out = torch.zeros_like(q)
    S = k.shape[0]
    key_pos = key_start + torch.arange(S)
    for a in range(0, q.shape[0], block):
        b = min(a + block, q.shape[0])
        first, last = int(q_pos[a]), int(q_pos[b - 1])
        lo = key_start
        if kind == "chunk":
            lo = max((first // size) * size, key_start)
        elif kind == "window":
            lo = max(first - size + 1, key_start)
        lo, hi = lo - key_start, min(last + 1 - key_start, S)
        mask = visible_mask(q_pos[a:b], kind, size, key_pos[lo:hi])
        out[a:b] = attention(q[a:b], k[lo:hi], v[lo:hi], mask)
    return out


# --------------------------------------------------------------------------- feed-forward


def silu(g: torch.Tensor) -> torch.Tensor:
    """crates/spite-models/src/llama/llama4.rs:266: g / (1 + exp(-g))."""
    return g / (1.0 + torch.exp(-g))


def swiglu_mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """crates/spite-models/src/llama/llama4.rs:257-271: down . (silu(gate.x) * (up.x)),
    weights ``[out, in]`` (dense.rs:189-197)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def router_top1(x: torch.Tensor, w_router: torch.Tensor, hints=None, hint_rel: float = 0.0, taken=None):
    """crates/spite-models/src/moe.rs:65-66,110-126: logits = W_r.x; pick by raw logit,
    descending, stable sort so that ties go to the lowest index; weight = sigmoid(logit).

    ``hints[t]`` (optional) names the expert that another implementation chose for row t.
    Where it differs from the choice made here and the two logits lie within ``hint_rel``
    times the size of the router's logits, the two experts are tied at that implementation's
    precision and the hint is followed (and counted in ``taken``); a hint further off is
    ignored.  The size is the root mean square of all logits of the call: the error of a logit
    that was computed from rounded inputs grows with the row's and the router's sizes, not with
    the logit's own value, which cancellation can make as small as the gap itself."""
    logits = x @ w_router.T
    E = logits.shape[-1]
    size = float(logits.pow(2).mean().sqrt())
    idx = torch.zeros(logits.shape[0], dtype=torch.int64)
    for t in range(logits.shape[0]):
        best = 0
        for e in range(1, E):
            if logits[t, e] > logits[t, best]:
                best = e
        if hints is not None and int(hints[t]) != best and 0 <= int(hints[t]) < E:
            gap = float(logits[t, best] - logits[t, int(hints[t])])
            if gap <= hint_rel * size:
                best = int(hints[t])
                if taken is not None:
                    taken.append(t)
        idx[t] = best
    chosen = logits.gather(1, idx[:, None])[:, 0]
    w = 1.0 / (1.0 + torch.exp(-chosen))
    return idx, w, logits


def moe_ffn(x, w_router, gate_up, down, sh_gate, sh_up, sh_down, hints=None, hint_rel=0.0, taken=None, chosen=None) -> torch.Tensor:
    """crates/spite-models/src/moe.rs:168-191 and llama4.rs:231-256.

    Routed: the expert's *input* is x*w (moe.rs:172-173), the output is not weighted
    (:188-191): y = D_e . (silu(G_e . xw) * (U_e . xw)).  Shared expert on the unscaled x,
    added (llama4.rs:253-255).  ``gate_up`` is ``[E, d, 2F]`` (gate = first F columns),
    ``down`` ``[E, F, d]``: the file layout, applied as x @ M.
    """
    idx, w, _ = router_top1(x, w_router, hints, hint_rel, taken)
    if chosen is not None:
        chosen.extend(idx.tolist())
    F_ = down.shape[1]
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        e = int(idx[t])
        xw = x[t] * w[t]
        gu = xw @ gate_up[e]
        a = silu(gu[:F_]) * gu[F_:]
        y[t] = a @ down[e]
    return y + swiglu_mlp(x, sh_gate, sh_up, sh_down)


# --------------------------------------------------------------------------- whole model


def layer_kinds(cfg: dict):
    """Which layers rotate and which have experts.

    Rotation: ``no_rope_layers[L] == 1`` means layer L rotates; absent, every fourth layer
    ((L+1) % 4 == 0) does not (crates/spite-models/src/llama/llama4.rs:94-95,155).
    Experts: (L+1) % interleave_moe_layer_step == 0 (llama4.rs:44-47)."""
    L = cfg["num_hidden_layers"]
    nr = cfg.get("no_rope_layers")
    if not nr:
        step = cfg.get("nope_layer_interval", 4)
        nr = [int((i + 1) % step != 0) for i in range(L)]
    moe_step = cfg.get("interleave_moe_layer_step", 1)
    moe = [moe_step > 0 and (i + 1) % moe_step == 0 for i in range(L)]
    return [bool(r) for r in nr], moe


def forward(cfg: dict, weights: dict, tokens, start_pos: int = 0, dtype=torch.float64,
            visibility: str | None = None, route_hints=None, hint_rel: float = 0.0, taken=None,
            chosen=None, rows=None, rope_angle_dtype=None) -> torch.Tensor:
    """Logits ``[T, V]`` of one whole sequence (crates/spite-models/src/llama/llama4.rs:74-283,
    layer-major instead of token-major; same arithmetic).  ``visibility`` of the rotating
    layers: ``chunk`` (configuration) or ``window`` (what the reference computes); default: the
    configuration's ``attention_local_kind``, else ``chunk``.  ``rows`` (ascending positions):
    logits ``[len(rows), V]`` of these positions only; the last layer then computes nothing
    else (every earlier layer feeds the keys of the next and stays whole).  ``rope_angle_dtype``:
    see ``apply_rope``."""
    if visibility is None:
        visibility = cfg.get("attention_local_kind", "chunk")
    W = {k: v.to(dtype) for k, v in weights.items()}
    d = cfg["hidden_size"]
    H = cfg["num_attention_heads"]
    G = cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or d // H
    eps = cfg.get("rms_norm_eps", 1e-5)
    C = cfg.get("attention_chunk_size")
    uses_rope, is_moe = layer_kinds(cfg)
    inv_freq = rope_inv_freq(hd, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    pairing = cfg.get("rope_pairing", "half")
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    T = tokens.shape[0]
    pos = torch.arange(start_pos, start_pos + T)

    h = W["model.embed_tokens.weight"][tokens]                      # llama4.rs:118-119
    n_layers = cfg["num_hidden_layers"]
    sel = None if rows is None else torch.as_tensor(list(rows), dtype=torch.int64) - start_pos
    for L in range(n_layers):
        p = f"model.layers.{L}."
        n = rms_norm(h, W[p + "input_layernorm.weight"], eps)       # :126-127
        k = (n @ W[p + "self_attn.k_proj.weight"].T).view(T, G, hd)  # :140-153
        v = (n @ W[p + "self_attn.v_proj.weight"].T).view(T, G, hd)
        last = L == n_layers - 1 and sel is not None
        if last:                                                    # only the wanted rows from here on
            h, n, qpos = h[sel], n[sel], pos[sel]
        else:
            qpos = pos
        q = (n @ W[p + "self_attn.q_proj.weight"].T).view(-1, H, hd)
        if uses_rope[L]:
            q = apply_rope(q, qpos, inv_freq, pairing, rope_angle_dtype)   # :157-160
            k = apply_rope(k, pos, inv_freq, pairing, rope_angle_dtype)
            if cfg.get("use_qk_norm", True):
                q = qk_l2_norm(q, eps)                              # :161-175
                k = qk_l2_norm(k, eps)
            kind, size = (visibility, C) if C else ("full", 0)
        else:
            if cfg.get("attn_temperature_tuning", True):
                s = attn_temperature(qpos, cfg.get("floor_scale", 8192), cfg.get("attn_scale", 0.1), dtype)
                q = q * s[:, None, None]                            # :178-183
            kind, size = "full", 0
        o = attention_rows(q, k, v, qpos, kind, size, start_pos).reshape(-1, H * hd)   # :198-201
        h = h + o @ W[p + "self_attn.o_proj.weight"].T              # :202-207
        n = rms_norm(h, W[p + "post_attention_layernorm.weight"], eps)  # :210-211
        f = p + "feed_forward."
        if is_moe[L]:
            took = []
            hints = None if route_hints is None else route_hints.get(L)
            if hints is not None and last:
                hints = [hints[int(i)] for i in sel]
            y = moe_ffn(n, W[f + "router.weight"], W[f + "experts.gate_up_proj"], W[f + "experts.down_proj"],
                        W[f + "shared_expert.gate_proj.weight"], W[f + "shared_expert.up_proj.weight"],
                        W[f + "shared_expert.down_proj.weight"],    # :212-256
                        hints, hint_rel, took, None if chosen is None else chosen.setdefault(L, []))
            if taken is not None:
                taken.extend((L, int(sel[t]) if last else t) for t in took)
        else:
            y = swiglu_mlp(n, W[f + "gate_proj.weight"], W[f + "up_proj.weight"], W[f + "down_proj.weight"])
        h = h + y                                                   # :272-274
    if sel is not None and n_layers == 0:
        h = h[sel]
    n = rms_norm(h, W["model.norm.weight"], eps)                    # :277-278
    head = W["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else W["lm_head.weight"]
    return n @ head.T                                               # :279


# --------------------------------------------------------------------------- sampling

LCG_MUL = 6364136223846793005
LCG_ADD = 1442695040888963407
MASK64 = (1 << 64) - 1


def lcg_next(state: int):
    """crates/spite-sampling/src/lib.rs:343-348: s <- s*6364136223846793005 + 1442695040888963407
    (wrapping); u = (s >> 33) / 2^31, a float32 in [0, 1)."""
    state = (state * LCG_MUL + LCG_ADD) & MASK64
    u = torch.tensor(float(state >> 33), dtype=torch.float32) / torch.tensor(2147483648.0, dtype=torch.float32)
    return state, float(u)


def greedy(logits: torch.Tensor) -> int:
    """Highest logit; on exact ties the lowest index.  (The reference's ``max_by``,
    crates/spite-sampling/src/lib.rs:236-243, returns the last of equal maxima; this
    engine defines the first, and the vector [0, 2, 1.95] -> 1 of
    crates/spite-executor/src/lib.rs:814-828 holds under both.)"""
    best = 0
    vals = logits.tolist()
    for i in range(1, len(vals)):
        if vals[i] > vals[best]:
            best = i
    return best


def apply_repetition_penalty(logits, context, penalty: float, repeat_last_n: int = 0):
    """crates/spite-sampling/src/lib.rs:206-232: over the last ``repeat_last_n`` tokens (0 =
    all), each distinct id once: l > 0 -> l/penalty, else l*penalty."""
    if abs(penalty - 1.0) < 1.1920929e-07 or logits.numel() == 0:
        return logits
    window = context if repeat_last_n == 0 or repeat_last_n >= len(context) else context[len(context) - repeat_last_n:]
    out = logits.clone()
    for t in set(int(x) for x in window):
        if 0 <= t < out.numel():
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def apply_temperature(logits, temperature: float):
    """crates/spite-sampling/src/lib.rs:116-125: l /= T when T > 0."""
    return logits if temperature <= 0 else logits / temperature


def apply_min_p(logits, min_p: float):
    """crates/spite-sampling/src/lib.rs:186-197: drop l < max + ln(min_p)."""
    if min_p <= 0:
        return logits
    thresh = logits.max() + math.log(min_p)
    return logits.masked_fill(logits < thresh, float("-inf"))


def apply_top_k(logits, k: int):
    """crates/spite-sampling/src/lib.rs:128-144: keep l >= the k-th largest value."""
    if k == 0 or k >= logits.numel():
        return logits
    thresh = torch.sort(logits, descending=True).values[k - 1]
    return logits.masked_fill(logits < thresh, float("-inf"))


def apply_top_p(logits, p: float):
    """crates/spite-sampling/src/lib.rs:147-180: sort by logit descending (stable), keep the
    shortest prefix whose mass/total >= p, at least one."""
    if p >= 1.0 or logits.numel() == 0:
        return logits
    vals = logits.to(torch.float32)
    order = sorted(range(vals.numel()), key=lambda i: -float(vals[i]))
    mx = float(vals[order[0]])
    total = float(torch.exp(vals - mx).sum())
    cum, kept = 0.0, 0
    for i in order:
        cum += math.exp(float(vals[i]) - mx)
        kept += 1
        if cum / total >= p:
            break
    out = logits.clone()
    for n, i in enumerate(order):
        if n >= max(kept, 1):
            out[i] = float("-inf")
    return out


def multinomial(logits: torch.Tensor, state: int):
    """crates/spite-sampling/src/lib.rs:247-265: m = max; total = sum exp(l-m); u = lcg;
    the first i with cumsum >= u*total (float32 running sum in index order); else argmax."""
    l32 = logits.to(torch.float32)
    m = l32.max()
    state, u = lcg_next(state)
    e = torch.exp(l32 - m)
    total = torch.tensor(0.0, dtype=torch.float32)
    for x in e:
        total = total + x
    target = torch.tensor(u, dtype=torch.float32) * total
    cum = torch.tensor(0.0, dtype=torch.float32)
    for i in range(e.numel()):
        cum = cum + e[i]
        if cum >= target:
            return i, state
    return greedy(l32), state


def sample(logits, context, state: int, temperature: float, top_k: int = 0, top_p: float = 1.0,
           min_p: float = 0.0, repetition_penalty: float = 1.0, repeat_last_n: int = 64):
    """crates/spite-sampling/src/lib.rs:273-296: penalty -> temperature -> min-p -> top-k ->
    top-p, then greedy when T <= 0 else multinomial."""
    l = logits.to(torch.float32).clone()
    l = apply_repetition_penalty(l, context, repetition_penalty, repeat_last_n)
    l = apply_temperature(l, temperature)
    l = apply_min_p(l, min_p)
    l = apply_top_k(l, top_k)
    l = apply_top_p(l, top_p)
    if temperature <= 0:
        return greedy(l), state
    return multinomial(l, state)
