"""Small Renanex configurations, model folders made from them, the plain model's logits, and a runner that feeds
requests through a loaded model step by step as a schedule says."""
from __future__ import annotations

import json
import os

import torch

from plain import renanex_plain as P


def attention(heads, kv, dim, vdim, size, keep, rot_dims, scale, v_mix=False, scaling=None, base=10000.0, ff=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "attention", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix,
                      "mask": {"size": size, "keep_first": keep}, "rot": rot}}


def mamba(inner, state, dt_rank, conv, ff=None):
    return {"type": "mamba1", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def lightning(heads, dim, vdim, decay, ff=None):
    return {"type": "lightning", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def model(width, vocab, layers, eps=1e-5, logit_scale=0.5, softcap=12.0):
    return {"architecture": "Renanex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "logit_softcap": softcap, "layers": layers}


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
CONFIGS = {
    # every mixer, two blending layers, a part-rotated head with scaled frequencies, a layer without feed-forward
    "mixed": model(64, 97, [
        attention(4, 2, 32, 16, 24, 3, 16, 1.2, v_mix=True, scaling=YARN, ff=80),
        mamba(96, 8, 5, 3, ff=48),
        lightning(2, 16, 24, [0.7, 0.97], ff=72),
        attention(8, 2, 16, 16, 40, 0, 16, 1.5, v_mix=True, ff=None),
        attention(2, 2, 16, 32, 1000, 0, 8, 0.9, v_mix=False, base=500.0, ff=64)]),
    # mixers with state only: no page is ever taken
    "stateful": model(48, 61, [lightning(3, 8, 16, [0.5, 0.9, 0.999], ff=40), mamba(56, 3, 1, 2, ff=None),
                               mamba(64, 20, 7, 5, ff=96)], eps=1e-6, logit_scale=1.0, softcap=0),
    # one key/value head under six heads, sizes that are no multiples of 16, a window shorter than a page and more
    # first tokens kept than a page holds
    "narrow": model(40, 50, [attention(6, 1, 24, 40, 8, 20, 24, 2.0, ff=56), lightning(1, 24, 8, [0.95], ff=None),
                             attention(3, 3, 8, 8, 19, 1, 4, 1.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 2.0},
                                       ff=24)], logit_scale=0.3, softcap=5.0),
}


def make_dir(tmp, name: str, seed: int = 0, sharpen: float = 1.0, dtype=torch.float32) -> str:
    """A model folder of random weights.  ``sharpen`` multiplies the weights of the query norms, so that the softmax
    is far from flat and a key that should not be seen, or is missing, shows in the logits."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights import write_random_model
    out = os.path.join(str(tmp), f"renanex_{name}_{seed}")
    write_random_model(dict(CONFIGS[name]), seed, out, dtype)
    path = os.path.join(out, "model.safetensors")
    w = load_file(path)
    for k in w:
        if k.endswith(".q.norm"):
            w[k] = (w[k].float() * sharpen).to(w[k].dtype)
        elif k.endswith((".mix.in", ".mix.x", ".mix.q", ".mix.k", ".mix.v", ".mix.g")) and "q.norm" not in k:
            w[k] = (w[k].float() * 8.0).to(w[k].dtype)  # activations of order one inside the recurrences
    save_file(w, path)
    return out


def read(model_dir: str):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return load_file(os.path.join(model_dir, "model.safetensors")), cfg


def tokens_of(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def plain_logits(model_dir: str, tokens, dtype=torch.float64) -> torch.Tensor:
    w, cfg = read(model_dir)
    return P.forward(w, cfg, tokens, dtype)


def run_schedule(lm, requests: dict, schedule) -> dict:
    """``requests``: id -> tokens; ``schedule``: steps, each a list of (id, count).  A request is admitted at its first
    entry and released after its last token.  Returns id -> logits at every position ``[n, vocab]``."""
    from machserve_amd.engine.step import StepEntry
    at, slots = {i: 0 for i in requests}, {}
    got = {i: [] for i in requests}
    for step in schedule:
        entries, order = [], []
        for i, count in step:
            if i not in slots:
                slots[i] = lm.cache.admit()
            entries.append(StepEntry(slots[i], requests[i][at[i]:at[i] + count], list(range(count))))
            order.append((i, count))
            at[i] += count
        logits = lm.step(entries).float().cpu()
        row = 0
        for i, count in order:
            got[i].append(logits[row:row + count].clone())
            row += count
        for i, _ in order:
            if at[i] == len(requests[i]) and i in slots:
                lm.cache.release(slots.pop(i))
    assert all(at[i] == len(requests[i]) for i in requests), "the schedule does not feed every token"
    return {i: torch.cat(v) for i, v in got.items()}


def relative_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: root mean square of the difference (mean taken off) over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()


def relative_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest row error."""
    return float(relative_errors(got, want).max())


def within(got: torch.Tensor, want: torch.Tensor, dtype) -> bool:
    """float32: every row within rounding of sums taken in another order (a key too many or too few, or a state that is
    lost, is off by 1e-2 and more).  bfloat16: rounding of activations grows through the layers and differs from row to
    row, so half the rows must be within 4e-2 and every row within 0.25 (logits that have nothing to do with the wanted
    ones are off by 1.4)."""
    e = relative_errors(got, want)
    if dtype == torch.float32:
        return float(e.max()) < 1e-4
    return float(e.median()) < 4e-2 and float(e.max()) < 0.25
