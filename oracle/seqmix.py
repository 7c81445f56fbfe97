"""Plain, slow torch-CPU statement of the sequence-mixer mechanisms (test infrastructure only; shares no code with
umbrella_amd/).  One function per mechanism, written from the equations, whole sequences at a time, in float64 unless
told otherwise.  Each takes plain tensors and numbers: no configuration objects, no cache, no batching.

Notation: n tokens, H query heads, G key/value heads, D key size, E value size, X the mixer's input [n, width].
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def group_rms_norm(x, w, groups: int, eps: float):
    """rows cut into `groups` equal consecutive parts, each divided by sqrt(mean(part^2) + eps); the row times w"""
    shape = x.shape
    parts = x.reshape(*shape[:-1], groups, shape[-1] // groups)
    parts = parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return parts.reshape(shape) * w


def unit_rms(x, eps: float):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def gated_ff(x, w_gate, w_up, w_down):
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def rotate_interleaved(x, positions, rot_dims: int, base: float):
    """x [n, heads, D]: features (2i, 2i+1), i < rot_dims / 2, turn by positions * base^(-2i / rot_dims); the rest pass"""
    out = x.clone()
    for i in range(rot_dims // 2):
        ang = positions.to(x.dtype) * (base ** (-2.0 * i / rot_dims))
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible_tokens(i: int, window: int):
    """token positions position i sees"""
    return [j for j in range(0, i + 1) if i - j < window]


def visible_blocks(i: int, window: int, pool: int):
    """pooled blocks position i sees: those that lie wholly before the window"""
    return [b for b in range(0, i // pool + 1) if b * pool + pool - 1 <= i - window]


def pooled_window_attention(X, wq, bq, wk, bk, wg, wo, bo, pos_bias, *, H, G, D, window, pool, rot_dims, base, scale, eps,
                            cache_round=None, pos0: int = 0):
    """Sliding-window attention with mean-pooled blocks and sigmoid weights; values are the projected keys.
    cache_round: optional function applied to what a cache would hold (keys after rotation and unit RMS, raw values),
    e.g. rounding to bfloat16, before they are pooled and attended.  Token t sits at position pos0 + t (pos0 > 0 only
    makes sense for tests of the position arithmetic: nothing before pos0 exists)."""
    n = X.shape[0]
    pos = torch.arange(pos0, pos0 + n)
    q = (X @ wq.T + bq).reshape(n, H, D)
    k = (X @ wk.T + bk).reshape(n, G, D)
    v = k.clone()
    q = unit_rms(rotate_interleaved(q, pos, rot_dims, base), eps)
    k = unit_rms(rotate_interleaved(k, pos, rot_dims, base), eps)
    if cache_round is not None:
        k, v = cache_round(k), cache_round(v)
    gate = torch.sigmoid(X @ wg.T)                                   # [n, H]
    out = torch.zeros(n, H, D, dtype=X.dtype)
    for t in range(n):
        i = pos0 + t
        toks = [j - pos0 for j in visible_tokens(i, window) if j >= pos0]
        blks = [b for b in visible_blocks(i, window, pool) if b * pool >= pos0]
        for h in range(H):
            g = h // (H // G)
            acc = torch.zeros(D, dtype=X.dtype)
            for b in blks:
                lo = b * pool - pos0
                kb, vb = k[lo:lo + pool, g].mean(0), v[lo:lo + pool, g].mean(0)
                acc += torch.sigmoid((q[t, h] @ kb) * scale + pos_bias[h]) * vb
            for j in toks:
                acc += torch.sigmoid((q[t, h] @ k[j, g]) * scale + pos_bias[h]) * v[j, g]
            out[t, h] = acc * gate[t, h]
    return out.reshape(n, H * D) @ wo.T + bo


def gated_linear_attention(X, wq, wk, wv, wg, wo, w_norm, wa1, wa2, ba2, *, H, D, E, tau, eps, state=None):
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q scaled by D^-1/2 and
    alpha = sigmoid(wa2 (wa1 x) + ba2)^(1/tau); per-head RMS norm of o times w_norm, times silu(wg x), then wo.
    Returns (output [n, width], final state [H, D, E])."""
    n = X.shape[0]
    q = (X @ wq.T).reshape(n, H, D) / math.sqrt(D)
    k = (X @ wk.T).reshape(n, H, D)
    v = (X @ wv.T).reshape(n, H, E)
    alpha = torch.sigmoid((X @ wa1.T) @ wa2.T + ba2).pow(1.0 / tau).reshape(n, H, D)
    S = torch.zeros(H, D, E, dtype=X.dtype) if state is None else state.clone()
    o = torch.zeros(n, H, E, dtype=X.dtype)
    for t in range(n):
        for h in range(H):
            S[h] = alpha[t, h][:, None] * S[h] + torch.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    o = unit_rms(o, eps) * w_norm
    return (o.reshape(n, H * E) * silu(X @ wg.T)) @ wo.T, S


def gitopel_forward(cfg: dict, sd: dict, tokens, dtype=F, cache_round=None, layers_out=None):
    """Whole-sequence forward of a Gitopel checkpoint: cfg is the parsed config.json, sd maps tensor names to tensors.
    Returns logits [n, vocab]."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in sd.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, ly in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ly["mixer"]
        h = group_rms_norm(x, w[p + "norm1"], groups, eps)
        if ly["type"] == "attention":
            y = pooled_window_attention(h, w[p + "mix.q"], w[p + "mix.q.b"], w[p + "mix.k"], w[p + "mix.k.b"], w[p + "mix.g"],
                                        w[p + "mix.o"], w[p + "mix.o.b"], w[p + "mix.pb"], H=m["heads"], G=m["kv_heads"],
                                        D=m["dim"], window=m["mask"]["size"], pool=m["mask"]["pool"], rot_dims=m["rot"]["dims"],
                                        base=m["rot"]["base"], scale=m["scale"], eps=eps, cache_round=cache_round)
        else:
            y, _ = gated_linear_attention(h, w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"], w[p + "mix.o"],
                                          w[p + "mix.norm"], w[p + "mix.a1"], w[p + "mix.a2"], w[p + "mix.a2.b"], H=m["heads"],
                                          D=m["dim"], E=m["vdim"], tau=m["tau"], eps=eps)
        x = x + group_rms_norm(y, w[p + "norm1b"], groups, eps)
        if ly.get("mlp") is not None:
            h = group_rms_norm(x, w[p + "norm2"], groups, eps)
            x = x + group_rms_norm(gated_ff(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"]), w[p + "norm2b"], groups, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return group_rms_norm(x, w["final.norm"], groups, eps) @ w["head"].T


# ---------------------------------------------------------------------------------------------------------------- Fidizen
def rms_norm(x, w, eps: float):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def conv_input(h, w, history=None):
    """What a sublayer reads: h[t] + sum_j w[:, j] * h[t - taps + 1 + j] (j = taps - 1 is h[t] itself), zeros before the
    start.  h [n, width], w [width, taps]; history: the inputs that came before h[0] (any number of rows, the last is
    h[-1])."""
    taps, n = w.shape[1], h.shape[0]
    past = torch.zeros(0, h.shape[1], dtype=h.dtype) if history is None else history
    full = torch.cat([past, h])
    off = past.shape[0]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            src = off + t - taps + 1 + j
            if src >= 0:
                out[t] = out[t] + w[:, j] * full[src]
    return out


def latent_attention(X, w_dq, n_dq, w_uq, w_dkv, n_dkv, w_uk, w_uv, sink, w_g, w_o, *, H, D, R, E, kv_rank, window, rot_dims,
                     base, scale, eps, cache_round=None, pos0: int = 0):
    """Softmax attention through latents.  c_q = norm(w_dq x), q = w_uq c_q laid out per head as [D unrotated | R rotated];
    w_dkv x = [kv_rank latent | R shared key part]; c = norm(latent); per head key = [w_uk c | rotated shared part], value =
    w_uv c.  Position i sees j with 0 <= i - j < window (window 0: all j <= i).  The softmax denominator also holds
    exp(sink[h]).  The heads, concatenated, are multiplied by sigmoid(w_g x) and go through w_o.
    cache_round: optional rounding of what a cache would hold (c and the rotated shared key part)."""
    n = X.shape[0]
    pos = torch.arange(pos0, pos0 + n)
    q = (rms_norm(X @ w_dq.T, n_dq, eps) @ w_uq.T).reshape(n, H, D + R)
    q_rot = rotate_interleaved(q[..., D:], pos, rot_dims, base)
    dkv = X @ w_dkv.T
    c = rms_norm(dkv[:, :kv_rank], n_dkv, eps)
    k_rot = rotate_interleaved(dkv[:, None, kv_rank:], pos, rot_dims, base)[:, 0]
    if cache_round is not None:
        c, k_rot = cache_round(c), cache_round(k_rot)
    k = (c @ w_uk.T).reshape(n, H, D)
    v = (c @ w_uv.T).reshape(n, H, E)
    out = torch.zeros(n, H, E, dtype=X.dtype)
    for t in range(n):
        lo = 0 if window <= 0 else max(0, t - window + 1)
        for h in range(H):
            s = (k[lo:t + 1, h] @ q[t, h, :D] + k_rot[lo:t + 1] @ q_rot[t, h]) * scale          # one score per visible j
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            p = e / (e.sum() + torch.exp(sink[h] - m))
            out[t, h] = (p[:, None] * v[lo:t + 1, h]).sum(0)
    return (out.reshape(n, H * E) * torch.sigmoid(X @ w_g.T)) @ w_o.T


def polynorm(z, coef, eps: float):
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3], N = unit RMS over the row"""
    return coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z * z, eps) + coef[2] * unit_rms(z * z * z, eps) + coef[3]


def routed_experts(X, w_router, experts, top: int, shared=None, margins=None):
    """experts: list of (w_gate, w_up, w_down).  score = sigmoid(router logit); the `top` largest (ties: lower index) are
    used, each expert fed score * x; outputs summed; `shared` (same triple) sees every token unweighted.
    margins: optional list that receives, per token, how far the last chosen logit lies above the first one not chosen, in
    units of the spread of that token's logits (tests pick inputs whose choices no rounding can flip)."""
    z = X @ w_router.T
    s = torch.sigmoid(z)
    out = torch.zeros_like(X)
    for t in range(X.shape[0]):
        # ranked on the logits: the same order as on the scores, also where the sigmoid has saturated to 1.0
        ranked = sorted(range(len(experts)), key=lambda e: (-float(z[t, e]), e))
        order = ranked[:top]
        if margins is not None and top < len(experts):
            margins.append(float((z[t, ranked[top - 1]] - z[t, ranked[top]]) / z[t].std().clamp_min(1e-30)))
        for e in order:
            out[t] = out[t] + gated_ff((s[t, e] * X[t])[None], *experts[e])[0]
    if shared is not None:
        out = out + gated_ff(X, *shared)
    return out


def fidizen_forward(cfg: dict, sd: dict, tokens, dtype=F, cache_round=None, layers_out=None, route_margins=None):
    """Whole-sequence forward of a Fidizen checkpoint: cfg is the parsed config.json, sd maps tensor names to tensors.
    Returns logits [n, vocab].  route_margins: see routed_experts."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, ly in enumerate(cfg["layers"]):
        p, m = f"l{ly.get('weights_of', i) if ly.get('weights_of') is not None else i}.", ly["mixer"]
        h = conv_input(x, w[p + "canon1"])
        y = latent_attention(h, w[p + "mix.dq"], w[p + "mix.dq.norm"], w[p + "mix.uq"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"],
                             w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.sink"], w[p + "mix.g"], w[p + "mix.o"], H=m["heads"],
                             D=m["dim"], R=m["rot_dim"], E=m["vdim"], kv_rank=m["kv_rank"], window=(m.get("mask") or {}).get("size", 0),
                             rot_dims=m["rot"]["dims"], base=m["rot"]["base"], scale=m["scale"], eps=eps, cache_round=cache_round)
        x = x + rms_norm(y, w[p + "norm1"], eps)
        mlp = ly.get("mlp")
        if mlp is not None:
            h = conv_input(x, w[p + "canon2"])
            if mlp["kind"] == "dense":
                y = polynorm(h @ w[p + "mlp.up"].T, w[p + "mlp.act"], eps) @ w[p + "mlp.down"].T
            else:
                ex = [tuple(w[p + f"mlp.e{e}.{n}"] for n in ("gate", "up", "down")) for e in range(mlp["router"]["experts"])]
                sh = tuple(w[p + f"mlp.shared.{n}"] for n in ("gate", "up", "down")) if mlp.get("shared") else None
                y = routed_experts(h, w[p + "mlp.router"], ex, mlp["router"]["top"], sh, margins=route_margins)
            x = x + rms_norm(y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
