"""Small Nubodra configurations, model folders made from them and the plain model's logits."""
from __future__ import annotations

import json
import os

import torch

from plain import nubodra_plain as P
from renanex_util import relative_error, relative_errors, run_schedule, tokens_of, within  # noqa: F401  (shared runners)


def conv_attention(heads, kv, dim, scale, conv=None, q_temp=None, ff=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if conv is not None:
        m["conv"] = conv
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=10000.0, scaling=None, kv_from=None, ff=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(width, vocab, layers, eps=1e-5, scale=2.5):
    return {"architecture": "Nubodra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale}, "layers": layers}


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
CONFIGS = {
    # both mixers twice, a layer that reads another's latent with heads and sizes of its own, a layer without feed-forward
    "pair": model(64, 97, [
        latent(4, 16, 8, 24, 40, 24, 0.3, scaling=YARN, ff=80),
        conv_attention(4, 2, 24, 0.25, conv=4, q_temp=(0.7, 5), ff=48),
        latent(2, 8, 8, 16, 16, 24, 0.5, scaling=YARN, kv_from=0, ff=72),
        conv_attention(3, 3, 16, 0.4, conv=2, q_temp=(0.2, 1), ff=None)]),
    # sizes that are no multiples of 8 or 16, one key/value head under six heads, five taps, two latent caches of
    # different widths, a rotation without scaling, an attention with one tap (no state) and no temperature
    "odd": model(48, 61, [
        conv_attention(6, 1, 20, 0.3, conv=5, q_temp=(1.5, 7), ff=40),
        latent(3, 12, 6, 20, 20, 26, 0.4, base=500.0, ff=None),
        latent(5, 8, 4, 8, 12, 12, 0.6, base=100.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 2.0}, ff=56),
        conv_attention(2, 2, 8, 0.7, conv=1, ff=24),
        latent(4, 4, 6, 6, 9, 26, 0.5, base=500.0, kv_from=1, ff=32)], eps=1e-6, scale=1.0),
    # heads of 64 numbers in both mixers (the attention kernels' tile of 64 takes work items of another size in the
    # two-byte types, so these heads run in the next tile), attention first, the temperature far beyond the prompts
    "sixtyfour": model(128, 128, [
        conv_attention(4, 4, 64, 0.15, conv=3, q_temp=(0.9, 4096), ff=96),
        latent(8, 32, 16, 64, 64, 48, 0.25, base=50000.0, scaling={"factor": 8.0, "original": 32, "fast": 16.0, "slow": 2.0}, ff=160),
        latent(2, 64, 16, 32, 32, 48, 0.2, base=50000.0, scaling={"factor": 8.0, "original": 32, "fast": 16.0, "slow": 2.0}, kv_from=1, ff=64),
        conv_attention(8, 2, 64, 0.1, conv=2, q_temp=(0.1, 2), ff=64)], eps=1e-6, scale=0.5),
    # more heads than a decode tile holds over one latent, more than a few heads a key/value head
    "heads": model(64, 80, [
        latent(20, 8, 8, 8, 32, 40, 0.5, ff=64),
        conv_attention(18, 1, 16, 0.3, conv=3, q_temp=(0.5, 16), ff=None),
        latent(17, 16, 8, 8, 24, 40, 0.4, kv_from=0, ff=48)], scale=4.0),
}


def make_dir(tmp, name: str, seed: int = 0, sharpen: float = 8.0, dtype=torch.float32) -> str:
    """A model folder of random weights.  ``sharpen`` multiplies the up projections of the latent layers' queries and keys
    and the rotated key part's rows, so that their softmax is far from flat (the other attention's scores are of order
    ``scale * sqrt(dim)`` already) and a key that is missing or one too many shows in the logits; the sinks are spread."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights import write_random_model
    out = os.path.join(str(tmp), f"nubodra_{name}_{seed}")
    write_random_model(dict(CONFIGS[name]), seed, out, dtype)
    path = os.path.join(out, "model.safetensors")
    w = load_file(path)
    g = torch.Generator().manual_seed(seed + 1)
    for i, layer in enumerate(CONFIGS[name]["layers"]):
        p = f"l{i}.mix."
        if layer["type"] == "latent_attention":
            r = layer["mixer"]["kv_rank"]
            for k in ("uq", "uk"):
                w[p + k] = (w[p + k].float() * sharpen).to(dtype)
            if p + "dkv" in w:
                t = w[p + "dkv"].float()
                t[r:] *= sharpen
                w[p + "dkv"] = t.to(dtype)
            w[p + "sink"] = (torch.randn(w[p + "sink"].shape, generator=g) * 1.5).to(dtype)
            w[p + "uv"] = (w[p + "uv"].float() * 4.0).to(dtype)
        else:
            w[p + "g"] = (w[p + "g"].float() * 30.0).to(dtype)   # gates away from one half
        w[f"l{i}.norm1.b"] = (torch.randn(w[f"l{i}.norm1.b"].shape, generator=g) * 0.3).to(dtype)
    save_file(w, path)
    return out


def read(model_dir: str):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return load_file(os.path.join(model_dir, "model.safetensors")), cfg


def plain_logits(model_dir: str, tokens, dtype=torch.float64, weights_as=None) -> torch.Tensor:
    """The plain model's logits; ``weights_as``: matrices rounded to this type first, as a run in that type holds them."""
    w, cfg = read(model_dir)
    if weights_as is not None and weights_as != torch.float32:
        w = {k: v.to(weights_as).float() if v.dim() == 2 and not k.endswith(".conv") else v for k, v in w.items()}
    return P.forward(w, cfg, tokens, dtype)
