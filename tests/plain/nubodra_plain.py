"""Plain, slow Nubodra decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Input is a dict of tensors by checkpoint name and the
config.json dict; everything is computed with ordinary torch operations on the CPU in
``dtype`` (float32 or float64).

Notation: ``n`` tokens, width ``w``; a linear map is ``y = x @ W.T`` with ``W [out, in]``.
"""
from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Rows divided by ``sqrt(mean(x^2) + eps)``."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ rotation
def rotary_frequencies(rot: dict):
    """``(freq [dims / 2] float64, factor)``: ``freq_i = base^(-2i / dims)``; with ``scaling`` a frequency goes over to
    ``1 / factor`` of itself along a ramp between two pair indices, and cosines and sines get ``0.1 ln(factor) + 1``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def index_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(index_of(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [n, ..., d]``: of the first ``dims`` numbers, neighbours ``(2i, 2i + 1)`` are rotated by ``position * freq_i``;
    the rest pass."""
    dims = int(rot["dims"])
    f, factor = rotary_frequencies(rot)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (torch.cos(ang) * factor).to(x.dtype).reshape(shape), (torch.sin(ang) * factor).to(x.dtype).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------ pieces of the mixers
def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``u [n, channels]``, ``w [channels, taps]``: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start."""
    n, taps = u.shape[0], w.shape[1]
    pad = torch.cat([u.new_zeros(taps - 1, u.shape[1]), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + n] * w[:, j]
    return y


def query_temperature(n: int, coef: float, every: int, dtype) -> torch.Tensor:
    """``[n]``: ``1 + coef ln(floor((p + 1) / every) + 1)``."""
    p = torch.arange(n, dtype=torch.float64)
    return (1.0 + coef * torch.log(torch.floor((p + 1.0) / every) + 1.0)).to(dtype)


def causal_softmax(scores: torch.Tensor, sink=None) -> torch.Tensor:
    """``scores [heads, n, n]``: softmax over the keys ``j <= i``; with ``sink [heads]`` the denominator also holds
    ``exp(sink)``: weight that goes to nothing."""
    n = scores.shape[-1]
    keep = torch.ones(n, n, dtype=torch.bool).tril()
    s = scores.masked_fill(~keep, float("-inf"))
    if sink is None:
        return torch.softmax(s, -1)
    full = torch.cat([s, sink.to(s.dtype)[:, None, None].expand(-1, n, 1)], -1)
    return torch.softmax(full, -1)[..., :n]


# ------------------------------------------------------------------ mixers
def attention(h, t, m, eps):
    """Grouped-query attention whose values are its keys: a short convolution after the q and k projections, values =
    keys before their unit norm, q and k of every head divided by their root mean square, a query temperature that
    grows with the position, and a sigmoid gate per head on the output."""
    n = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q, k = h @ t["q"].T, h @ t["k"].T
    if m.get("conv"):
        q, k = causal_conv(q, t["q.conv"]), causal_conv(k, t["k.conv"])
    q, k = q.view(n, H, d), k.view(n, G, d)
    v = k
    q, k = rms(q, eps), rms(k, eps)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(n, float(qt["coef"]), int(qt["every"]), q.dtype)[:, None, None]
    k_of = torch.arange(H) // (H // G)
    s = torch.einsum("ihd,jhd->hij", q, k[:, k_of]) * float(m["scale"])
    p = causal_softmax(s)
    o = torch.einsum("hij,jhd->ihd", p, v[:, k_of])
    o = o * torch.sigmoid(h @ t["g"].T)[:, :, None]
    return o.reshape(n, -1) @ t["o"].T


def latent_of(h, t, m, eps):
    """What a latent-attention layer keeps of a token: ``(c [n, kv_rank], rotated key part [n, rot_dim])``."""
    r = m["kv_rank"]
    dkv = h @ t["dkv"].T
    c = rms(dkv[:, :r], eps) * t["dkv.norm"]
    kr = rotate_interleaved(dkv[:, r:], torch.arange(h.shape[0]), m["rot"])
    return c, kr


def latent_attention(h, t, m, eps, latent):
    """Attention through a latent: queries from a normed bottleneck, keys ``[W_uk c | shared rotated part]``, values
    ``W_uv c``, a sink in the softmax.  ``latent``: ``(c, rotated key part)`` of this layer or of the one it reads."""
    n = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = latent
    cq = rms(h @ t["dq"].T, eps) * t["dq.norm"]
    q = (cq @ t["uq"].T).view(n, H, d + dr)
    qn, qr = q[..., :d], rotate_interleaved(q[..., d:], torch.arange(n), m["rot"])
    kn = (c @ t["uk"].T).view(n, H, d)
    v = (c @ t["uv"].T).view(n, H, dv)
    s = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * float(m["scale"])
    p = causal_softmax(s, t["sink"])
    o = torch.einsum("hij,jhd->ihd", p, v)
    return o.reshape(n, -1) @ t["o"].T


def feed_forward(h, t):
    return (silu(h @ t["gate"].T) * (h @ t["up"].T)) @ t["down"].T


# ------------------------------------------------------------------ the model
def _sub(tensors, prefix, dtype):
    return {k[len(prefix):]: v.to(dtype) for k, v in tensors.items() if k.startswith(prefix)}


def forward(tensors, cfg, tokens, dtype=torch.float64, streams=None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of one sequence.  ``streams``: a list that receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = tensors["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)] * float(cfg.get("embedding", {}).get("scale", 1.0))
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        m, t = layer["mixer"], _sub(tensors, f"l{i}.mix.", dtype)
        h = layer_norm(x, tensors[f"l{i}.norm1"].to(dtype), tensors[f"l{i}.norm1.b"].to(dtype), eps)
        if layer["type"] == "attention":
            y = attention(h, t, m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_of(h, t, m, eps)
                src = i
            y = latent_attention(h, t, m, eps, latents[src])
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        if layer.get("mlp") is not None:
            y = y + feed_forward(h, _sub(tensors, f"l{i}.mlp.", dtype))
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    x = layer_norm(x, tensors["final.norm"].to(dtype), tensors["final.norm.b"].to(dtype), eps)
    return x @ tensors["head"].to(dtype).T


def greedy_generate(tensors, cfg, prompt, n_new: int, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(tensors, cfg, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]
