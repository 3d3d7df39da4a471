"""Plain, slow Renanex decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Input is a dict of tensors by checkpoint name and the
config.json dict; everything is computed with ordinary torch operations on the CPU in
``dtype`` (float32 or float64), token after token where the mechanism is a recurrence.

Notation: ``n`` tokens, width ``w``; a linear map is ``y = x @ W.T`` with ``W [out, in]``.
"""
from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Rows divided by ``sqrt(mean(x^2) + eps)``."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ rotation
def rotary_frequencies(rot: dict, dtype=torch.float64):
    """``(freq [dims / 2], factor)``: ``freq_i = base^(-2i / dims)``; with ``scaling`` a frequency goes over to
    ``1 / factor`` of itself along a ramp between two pair indices, and cosines and sines get the factor
    ``0.1 ln(factor) + 1``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f.to(dtype), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def index_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(index_of(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(dtype), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [n, heads, dim]``: the first ``dims`` numbers of each head are rotated in pairs ``(i, i + dims / 2)`` by the
    angle ``position * freq_i``; the rest pass."""
    dims = int(rot["dims"])
    f, factor = rotary_frequencies(rot, x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * factor)[:, None, :], (torch.sin(ang) * factor)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ------------------------------------------------------------------ mixers
def visible(n: int, size: int, keep_first: int) -> torch.Tensor:
    """``[n, n]`` bool: row i sees column j if ``j <= i`` and (``i - j < size`` or ``j < keep_first``)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def attention(h, t, m, eps, v_first=None):
    """Grouped-query attention with a norm over the whole q and k projections, partial rotation, scores mixed between
    the heads before the softmax, a window that keeps the first tokens, and values blended with those of the first
    such layer.  ``t``: the mixer's tensors by their short names.  Returns ``(output [n, w], values [n, kv * vdim])``;
    the values are the layer's own before blending if ``v_first`` is None, else the blended ones."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ t["q"].T, eps) * t["q.norm"]
    k = rms(h @ t["k"].T, eps) * t["k.norm"]
    v = h @ t["v"].T
    if m.get("v_mix") and v_first is not None:
        lam = t["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    pos = torch.arange(n)
    q = rotate(q.view(n, H, d), pos, m["rot"])
    k = rotate(k.view(n, G, d), pos, m["rot"])
    vv = v.view(n, G, dv)
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1)            # query head h reads key/value head h // rep
    vh = vv.repeat_interleave(rep, dim=1)
    score = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]
    score = torch.einsum("hg,gij->hij", t["talk"], score)
    mask = visible(n, m["mask"]["size"], m["mask"]["keep_first"])
    score = score.masked_fill(~mask[None], float("-inf"))
    w = torch.softmax(score, -1)
    o = torch.einsum("hij,jhe->ihe", w, vh).reshape(n, H * dv)
    return o @ t["o"].T, v


def lightning(h, t, m, eps):
    """Linear attention with a decay per head: ``S <- decay * S + k v^T``, ``o = S^T q``, token after token; the heads'
    outputs are normed together, gated and projected."""
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ t["q"].T).view(n, H, d)
    k = silu(h @ t["k"].T).view(n, H, d)
    v = silu(h @ t["v"].T).view(n, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    o = torch.empty(n, H, dv, dtype=h.dtype)
    for i in range(n):
        S = decay[:, None, None] * S + k[i][:, :, None] * v[i][:, None, :]
        o[i] = torch.einsum("hde,hd->he", S, q[i])
    y = rms(o.reshape(n, H * dv), eps) * t["norm"] * torch.sigmoid(h @ t["g"].T)
    return y @ t["o"].T


def mamba1(h, t, m):
    """Selective scan: a short causal convolution, then per channel and state ``S <- exp(dt A) S + dt x B``,
    ``y = S . C + D x``, gated by ``silu(z)``."""
    n = h.shape[0]
    C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ t["in"].T
    x, z = xz[:, :C], xz[:, C:]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=h.dtype), x], 0)
    conv = torch.zeros_like(x)
    for k in range(taps):                      # the last column of the filter meets the current token
        conv = conv + padded[k:k + n] * t["conv"][:, k]
    x = silu(conv + t["conv.b"])
    dbc = x @ t["x"].T
    dt = softplus(dbc[:, :R] @ t["dt"].T + t["dt.b"])
    B, Cm = dbc[:, R:R + N], dbc[:, R + N:R + 2 * N]
    A = -torch.exp(t["A_log"])
    S = torch.zeros(C, N, dtype=h.dtype)
    y = torch.empty(n, C, dtype=h.dtype)
    for i in range(n):
        S = torch.exp(dt[i][:, None] * A) * S + (dt[i] * x[i])[:, None] * B[i][None, :]
        y[i] = S @ Cm[i] + t["D"] * x[i]
    return (y * silu(z)) @ t["o"].T


def feed_forward(h, t):
    return (silu(h @ t["gate"].T) * (h @ t["up"].T)) @ t["down"].T


# ------------------------------------------------------------------ the model
def _sub(weights, prefix, dtype):
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def forward(weights, cfg, tokens, dtype=torch.float64, layers_out=None):
    """Logits ``[n, vocab]`` of a whole sequence.  ``layers_out``: a list that receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)]
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        g = {k: weights[p + k].to(dtype) for k in ("norm1", "norm1b", "norm2", "norm2b") if p + k in weights}
        t, m = _sub(weights, p + "mix.", dtype), layer["mixer"]
        h = rms(x, eps) * g["norm1"]
        if layer["type"] == "attention":
            y, v = attention(h, t, m, eps, v_first if m.get("v_mix") else None)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "lightning":
            y = lightning(h, t, m, eps)
        elif layer["type"] == "mamba1":
            y = mamba1(h, t, m)
        else:
            raise ValueError(f"no mixer {layer['type']!r}")
        x = x + rms(y, eps) * g["norm1b"]
        if layer.get("mlp"):
            y = feed_forward(rms(x, eps) * g["norm2"], _sub(weights, p + "mlp.", dtype))
            x = x + rms(y, eps) * g["norm2b"]
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rms(x, eps) * weights["final.norm"].to(dtype)
    logits = (h @ weights["head"].to(dtype).T) * float(cfg.get("logit_scale", 1.0))
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy_generate(weights, cfg, prompt, max_new, dtype=torch.float64):
    seq = list(prompt)
    for _ in range(max_new):
        seq.append(int(forward(weights, cfg, seq, dtype)[-1].argmax()))
    return seq[len(prompt):]
