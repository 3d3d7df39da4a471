"""Typed configuration of the Renanex decoder, read from config.json's own keys.

A Renanex model is a list of layers, each with one mixer - ``mamba1`` (a selective scan), ``attention``
(grouped-query attention whose heads exchange scores, over a window that keeps the first tokens) or
``lightning`` (linear attention with a decay per head) - and an optional dense gated feed-forward, every branch
between two RMS norms whose weight is a single number.  The logits are scaled and then capped by a tanh.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``logit_scale``, ``logit_softcap``, and ``layers``, a
list of ``{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}``.  Every size and constant comes from
there; a missing or ill-typed key is an error that names it.  Tensor names: ``embed``, ``head``, ``final.norm``,
and per layer ``l<i>.norm1 | norm1b | norm2 | norm2b``, ``l<i>.mix.*`` and ``l<i>.mlp.gate | up | down``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .specs import (ConfigError, EmbeddingSpec, GatedMlpSpec, HeadSpec, LightningSpec, ModelSpec, NormSpec, RotarySpec,
                    SandwichLayerSpec, SelectiveScanSpec, TalkingAttentionSpec, YarnSpec)

ARCHITECTURE = "Renanex"
# the configuration names no longest sequence: positions are 32-bit integers, and the pools bound a request
MAX_POSITIONS = 1 << 30


def _get(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: missing key '{where}{key}'")
    return d[key]


def _int(d: dict, key: str, where: str, minimum: int = 1) -> int:
    v = _get(d, key, where)
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError(f"config.json: '{where}{key}' must be an integer >= {minimum}, got {v!r}")
    return v


def _num(d: dict, key: str, where: str, positive: bool = True) -> float:
    v = _get(d, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and v <= 0):
        raise ConfigError(f"config.json: '{where}{key}' must be a{' positive' if positive else ''} number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[float, int, float, float]]  # factor, original, fast, slow


@dataclass(frozen=True)
class AttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    keep_first: int
    rot: RotationConfig
    v_mix: bool
    type: str = "attention"


@dataclass(frozen=True)
class Mamba1Layer:
    inner: int
    state: int
    dt_rank: int
    conv: int
    type: str = "mamba1"


@dataclass(frozen=True)
class LightningLayer:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    type: str = "lightning"


def _mixer_of(kind: str, m: dict, where: str):
    if kind == "attention":
        heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: '{where}heads' {heads} is not a multiple of '{where}kv_heads' {kv}")
        dim = _int(m, "dim", where)
        mask = m.get("mask")  # none: every earlier token is seen
        rot = m.get("rot") or {"dims": 0, "base": 10000.0}  # none: nothing is rotated
        dims = _int(rot, "dims", where + "rot.", 0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"config.json: '{where}rot.dims' {dims} must be even and at most '{where}dim' {dim}")
        sc = rot.get("scaling")
        scaling = None
        if sc is not None:
            w = where + "rot.scaling."
            scaling = (_num(sc, "factor", w), int(_num(sc, "original", w)), _num(sc, "fast", w), _num(sc, "slow", w))
        return AttentionLayer(heads, kv, dim, _int(m, "vdim", where), _num(m, "scale", where),
                              _int(mask, "size", where + "mask.") if mask is not None else None,
                              _int(mask, "keep_first", where + "mask.", 0) if mask is not None and mask.get("keep_first") is not None else 0,
                              RotationConfig(_num(rot, "base", where + "rot."), dims, scaling), bool(m.get("v_mix", False)))
    if kind == "mamba1":
        return Mamba1Layer(_int(m, "inner", where), _int(m, "state", where), _int(m, "dt_rank", where), _int(m, "conv", where))
    if kind == "lightning":
        heads = _int(m, "heads", where)
        decay = _get(m, "decay", where)
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay):
            raise ConfigError(f"config.json: '{where}decay' must list one number for each of the {heads} heads, got {decay!r}")
        return LightningLayer(heads, _int(m, "dim", where), _int(m, "vdim", where), tuple(float(v) for v in decay))
    raise ConfigError(f"config.json: '{where[:-6]}type' {kind!r} is not a mixer of this architecture (attention, lightning, mamba1)")


@dataclass(frozen=True)
class RenanexConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    logit_softcap: float   # 0: no cap
    mixers: tuple          # one of AttentionLayer, Mamba1Layer, LightningLayer per layer
    ff: tuple              # per layer the feed-forward's size, or None

    @classmethod
    def from_dict(cls, raw: dict) -> "RenanexConfig":
        layers = _get(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        mixers, ff = [], []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: 'layers[{i}]' must be an object")
            kind = _get(layer, "type", where)
            mixers.append(_mixer_of(kind, _get(layer, "mixer", where), where + "mixer."))
            mlp = layer.get("mlp")
            if mlp is None:
                ff.append(None)
            else:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: '{where}mlp.kind' {mlp.get('kind')!r} is not supported (dense)")
                ff.append(_int(mlp, "ff", where + "mlp."))
        blend = [m for m in mixers if isinstance(m, AttentionLayer) and m.v_mix]
        if any((m.kv_heads, m.vdim) != (blend[0].kv_heads, blend[0].vdim) for m in blend):
            raise ConfigError("config.json: the layers with 'v_mix' must have the same 'kv_heads' and 'vdim'")
        cap = raw.get("logit_softcap")
        return cls(vocab=_int(raw, "vocab", ""), width=_int(raw, "width", ""), norm_eps=_num(_get(raw, "norm", ""), "eps", "norm."),
                   logit_scale=_num(raw, "logit_scale", "") if raw.get("logit_scale") is not None else 1.0,
                   logit_softcap=_num(raw, "logit_softcap", "") if cap else 0.0, mixers=tuple(mixers), ff=tuple(ff))

    # ------------------------------------------------------------------ back to config.json
    def to_dict(self) -> dict:
        layers = []
        for m, ff in zip(self.mixers, self.ff):
            if isinstance(m, AttentionLayer):
                rot = {"base": m.rot.base, "dims": m.rot.dims}
                if m.rot.scaling is not None:
                    f, o, fast, slow = m.rot.scaling
                    rot["scaling"] = {"factor": f, "original": o, "fast": fast, "slow": slow}
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "rot": rot, "v_mix": m.v_mix}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window, "keep_first": m.keep_first}
            elif isinstance(m, Mamba1Layer):
                mixer = {"inner": m.inner, "state": m.state, "dt_rank": m.dt_rank, "conv": m.conv}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay)}
            layers.append({"type": m.type, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}})
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap, "layers": layers}

    # ------------------------------------------------------------------ the model as data
    def _norm(self, name: str) -> NormSpec:
        return NormSpec("rmsnorm_scalar", self.width, self.norm_eps, {"weight": name})

    def to_spec(self) -> ModelSpec:
        layers = []
        first_blend = next((i for i, m in enumerate(self.mixers) if isinstance(m, AttentionLayer) and m.v_mix), None)
        for i, (m, ff) in enumerate(zip(self.mixers, self.ff)):
            p = f"l{i}.mix."
            if isinstance(m, AttentionLayer):
                yarn = None
                if m.rot.scaling is not None:
                    f, o, fast, slow = m.rot.scaling
                    yarn = YarnSpec(f, o, fast, slow)
                rotary = (RotarySpec("rotary", m.dim, m.rot.base, yarn=yarn, rotary_dim=m.rot.dims, table_precision="float64")
                          if m.rot.dims > 0 else None)
                mixer = TalkingAttentionSpec(
                    "talking_attention", self.width, m.heads, m.kv_heads, m.dim, m.vdim, rotary, m.scale, window=m.window,
                    keep_first=m.keep_first, qk_norm=True, norm_eps=self.norm_eps, talk=True,
                    value_blend=None if not m.v_mix else ("source" if i == first_blend else "blend"),
                    tensors={"q.weight": p + "q", "k.weight": p + "k", "v.weight": p + "v", "o.weight": p + "o",
                             "q_norm.weight": p + "q.norm", "k_norm.weight": p + "k.norm", "talk": p + "talk", "blend": p + "vmix"})
            elif isinstance(m, Mamba1Layer):
                mixer = SelectiveScanSpec(
                    "mamba1", self.width, m.inner, m.state, m.dt_rank, m.conv,
                    tensors={"in.weight": p + "in", "conv.weight": p + "conv", "conv.bias": p + "conv.b", "x.weight": p + "x",
                             "dt.weight": p + "dt", "dt.bias": p + "dt.b", "A_log": p + "A_log", "D": p + "D", "o.weight": p + "o"})
            else:
                mixer = LightningSpec(
                    "lightning", self.width, m.heads, m.dim, m.vdim, m.decay, self.norm_eps,
                    tensors={"q.weight": p + "q", "k.weight": p + "k", "v.weight": p + "v", "g.weight": p + "g", "o.weight": p + "o",
                             "norm.weight": p + "norm"})
            feed = None
            if ff is not None:
                q = f"l{i}.mlp."
                feed = GatedMlpSpec("gated_mlp", self.width, ff, "silu",
                                    tensors={"gate.weight": q + "gate", "up.weight": q + "up", "down.weight": q + "down"})
            layers.append(SandwichLayerSpec("sandwich", mixer, feed, self._norm(f"l{i}.norm1"), self._norm(f"l{i}.norm1b"),
                                            self._norm(f"l{i}.norm2") if feed else None, self._norm(f"l{i}.norm2b") if feed else None))
        spec = ModelSpec(
            architecture=ARCHITECTURE, embedding=EmbeddingSpec(self.vocab, self.width, {"weight": "embed"}), layers=tuple(layers),
            order=tuple(range(len(layers))), final_norm=self._norm("final.norm"),
            head=HeadSpec(self.vocab, self.width, False, {"weight": "head"}, scale=self.logit_scale, softcap=self.logit_softcap),
            max_positions=MAX_POSITIONS)
        spec.validate()
        return spec

    # ------------------------------------------------------------------ random weights
    def random_tensor_plan(self):
        """(name, shape, law) of every tensor of a random checkpoint; the laws are those of ``weights.random_init``."""
        w = self.width
        plan = [("embed", (self.vocab, w), "matrix")]
        for i, (m, ff) in enumerate(zip(self.mixers, self.ff)):
            plan += [(f"l{i}.norm1", (), "norm"), (f"l{i}.norm1b", (), "norm")]
            if ff is not None:
                plan += [(f"l{i}.norm2", (), "norm"), (f"l{i}.norm2b", (), "norm")]
            p = f"l{i}.mix."
            if isinstance(m, AttentionLayer):
                plan += [(p + "q", (m.heads * m.dim, w), "matrix"), (p + "k", (m.kv_heads * m.dim, w), "matrix"),
                         (p + "v", (m.kv_heads * m.vdim, w), "matrix"), (p + "q.norm", (m.heads * m.dim,), "norm"),
                         (p + "k.norm", (m.kv_heads * m.dim,), "norm"), (p + "talk", (m.heads, m.heads), "mixing"),
                         (p + "o", (w, m.heads * m.vdim), "matrix")]
                if m.v_mix:
                    plan.append((p + "vmix", (), "blend"))
            elif isinstance(m, Mamba1Layer):
                plan += [(p + "in", (2 * m.inner, w), "matrix"), (p + "conv", (m.inner, m.conv), "filter"), (p + "conv.b", (m.inner,), "bias"),
                         (p + "x", (m.dt_rank + 2 * m.state, m.inner), "matrix"), (p + "dt", (m.inner, m.dt_rank), "filter"),
                         (p + "dt.b", (m.inner,), "step_bias"), (p + "A_log", (m.inner, m.state), "a_log"), (p + "D", (m.inner,), "norm"),
                         (p + "o", (w, m.inner), "matrix")]
            else:
                plan += [(p + "q", (m.heads * m.dim, w), "matrix"), (p + "k", (m.heads * m.dim, w), "matrix"),
                         (p + "v", (m.heads * m.vdim, w), "matrix"), (p + "g", (m.heads * m.vdim, w), "matrix"),
                         (p + "o", (w, m.heads * m.vdim), "matrix"), (p + "norm", (m.heads * m.vdim,), "norm")]
            if ff is not None:
                q = f"l{i}.mlp."
                plan += [(q + "gate", (ff, w), "matrix"), (q + "up", (ff, w), "matrix"), (q + "down", (w, ff), "matrix")]
        plan += [("final.norm", (), "norm"), ("head", (self.vocab, w), "matrix")]
        return plan
