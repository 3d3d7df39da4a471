"""Typed configuration of the Nubodra decoder, read from config.json's own keys.

A Nubodra model is a list of parallel layers: one layer norm (weight and bias) feeds a mixer and an optional dense
gated feed-forward, and both are added to the stream.  The mixer is ``attention`` (grouped-query attention whose values
are its keys, behind a short convolution, with unit-normed q and k, a query temperature and a sigmoid gate per head)
or ``latent_attention`` (queries through a normed bottleneck, keys and values from a cached latent plus one rotated
key part shared by the heads, a sink in the softmax; ``kv_from`` names the layer whose cache a layer reads instead of
writing one).  The embedding is scaled; the output is a layer norm and a linear head.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, and ``layers``, a list of
``{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}``.  Every size and constant comes from there; a
missing or ill-typed key is an error that names it.  Tensor names: ``embed``, ``head``, ``final.norm`` (+ ``.b``), and
per layer ``l<i>.norm1`` (+ ``.b``), ``l<i>.mix.*`` and ``l<i>.mlp.gate | up | down``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .renanex import RotationConfig, _get, _int, _num
from .specs import (ConfigError, ConvAttentionSpec, EmbeddingSpec, GatedMlpSpec, HeadSpec, LatentAttentionSpec, ModelSpec,
                    NormSpec, ParallelLayerSpec, RotarySpec, YarnSpec)

ARCHITECTURE = "Nubodra"
# the configuration names no longest sequence: positions are 32-bit integers, and the pools bound a request
MAX_POSITIONS = 1 << 30


@dataclass(frozen=True)
class ConvAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    conv: int                              # taps of the convolution; 0: none
    q_temp: Optional[Tuple[float, int]]    # (coef, every) or None
    type: str = "attention"


@dataclass(frozen=True)
class LatentAttentionLayer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Optional[RotationConfig]
    kv_from: Optional[int]
    type: str = "latent_attention"


def _mixer_of(kind: str, m: dict, where: str):
    if kind == "attention":
        heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: '{where}heads' {heads} is not a multiple of '{where}kv_heads' {kv}")
        dim = _int(m, "dim", where)
        if m.get("vdim") is not None and _int(m, "vdim", where) != dim:
            raise ConfigError(f"config.json: '{where}vdim' {m['vdim']} differs from '{where}dim' {dim}, but the values are the keys")
        conv = _int(m, "conv", where, 1) if m.get("conv") is not None else 0
        qt = m.get("q_temp")
        q_temp = None
        if qt is not None:
            q_temp = (_num(qt, "coef", where + "q_temp.", positive=False), _int(qt, "every", where + "q_temp."))
        return ConvAttentionLayer(heads, kv, dim, _num(m, "scale", where), conv, q_temp)
    if kind == "latent_attention":
        rot_dim = _int(m, "rot_dim", where, 0)
        rot = None
        if rot_dim > 0:
            r = _get(m, "rot", where)
            dims = _int(r, "dims", where + "rot.", 2)
            if dims != rot_dim or dims % 2:
                raise ConfigError(f"config.json: '{where}rot.dims' {dims} must be even and equal to '{where}rot_dim' {rot_dim}")
            sc = r.get("scaling")
            scaling = None
            if sc is not None:
                w = where + "rot.scaling."
                scaling = (_num(sc, "factor", w), int(_num(sc, "original", w)), _num(sc, "fast", w), _num(sc, "slow", w))
            rot = RotationConfig(_num(r, "base", where + "rot."), dims, scaling)
        src = m.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or src < 0):
            raise ConfigError(f"config.json: '{where}kv_from' must be a layer's index, got {src!r}")
        return LatentAttentionLayer(_int(m, "heads", where), _int(m, "dim", where), rot_dim, _int(m, "vdim", where),
                                    _int(m, "q_rank", where), _int(m, "kv_rank", where), _num(m, "scale", where), rot, src)
    raise ConfigError(f"config.json: '{where[:-6]}type' {kind!r} is not a mixer of this architecture (attention, latent_attention)")


@dataclass(frozen=True)
class NubodraConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    mixers: tuple          # one of ConvAttentionLayer, LatentAttentionLayer per layer
    ff: tuple              # per layer the feed-forward's size, or None

    @classmethod
    def from_dict(cls, raw: dict) -> "NubodraConfig":
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
        for i, m in enumerate(mixers):
            src = getattr(m, "kv_from", None)
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if src >= i or not isinstance(mixers[src], LatentAttentionLayer) or mixers[src].kv_from is not None:
                raise ConfigError(f"config.json: '{where}' {src} must name an earlier latent_attention layer with a cache of its own")
            o = mixers[src]
            if (o.kv_rank, o.rot_dim, o.rot) != (m.kv_rank, m.rot_dim, m.rot):
                raise ConfigError(f"config.json: '{where}' {src}: the two layers' kv_rank, rot_dim and rot differ")
        emb = raw.get("embedding") or {}
        return cls(vocab=_int(raw, "vocab", ""), width=_int(raw, "width", ""), norm_eps=_num(_get(raw, "norm", ""), "eps", "norm."),
                   embedding_scale=_num(emb, "scale", "embedding.", positive=False) if emb.get("scale") is not None else 1.0,
                   mixers=tuple(mixers), ff=tuple(ff))

    # ------------------------------------------------------------------ back to config.json
    def to_dict(self) -> dict:
        layers = []
        for m, ff in zip(self.mixers, self.ff):
            if isinstance(m, ConvAttentionLayer):
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.dim, "scale": m.scale}
                if m.conv:
                    mixer["conv"] = m.conv
                if m.q_temp is not None:
                    mixer["q_temp"] = {"coef": m.q_temp[0], "every": m.q_temp[1]}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank,
                         "scale": m.scale}
                if m.rot is not None:
                    mixer["rot"] = {"base": m.rot.base, "dims": m.rot.dims}
                    if m.rot.scaling is not None:
                        f, o, fast, slow = m.rot.scaling
                        mixer["rot"]["scaling"] = {"factor": f, "original": o, "fast": fast, "slow": slow}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            layers.append({"type": m.type, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}})
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embedding_scale}, "layers": layers}

    # ------------------------------------------------------------------ the model as data
    def _norm(self, name: str) -> NormSpec:
        return NormSpec("layernorm", self.width, self.norm_eps, {"weight": name, "bias": name + ".b"})

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, (m, ff) in enumerate(zip(self.mixers, self.ff)):
            p = f"l{i}.mix."
            if isinstance(m, ConvAttentionLayer):
                mixer = ConvAttentionSpec(
                    "conv_attention", self.width, m.heads, m.kv_heads, m.dim, m.scale, conv_taps=m.conv, unit_norm=True,
                    norm_eps=self.norm_eps, q_temp=m.q_temp, gate=True,
                    tensors={"q.weight": p + "q", "k.weight": p + "k", "q.conv": p + "q.conv", "k.conv": p + "k.conv", "g.weight": p + "g",
                             "o.weight": p + "o"})
            else:
                rotary = None
                if m.rot is not None:
                    yarn = None
                    if m.rot.scaling is not None:
                        f, o, fast, slow = m.rot.scaling
                        yarn = YarnSpec(f, o, fast, slow)
                    rotary = RotarySpec("rotary", m.rot_dim, m.rot.base, yarn=yarn, rotary_dim=m.rot.dims, table_precision="float64",
                                        pairing="neighbours")
                mixer = LatentAttentionSpec(
                    "latent_attention", self.width, m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank, m.scale, rotary,
                    norm_eps=self.norm_eps, sink=True, kv_source=m.kv_from,
                    tensors={"dq.weight": p + "dq", "dq.norm": p + "dq.norm", "uq.weight": p + "uq", "dkv.weight": p + "dkv",
                             "dkv.norm": p + "dkv.norm", "uk.weight": p + "uk", "uv.weight": p + "uv", "sink": p + "sink", "o.weight": p + "o"})
            feed = None
            if ff is not None:
                q = f"l{i}.mlp."
                feed = GatedMlpSpec("gated_mlp", self.width, ff, "silu",
                                    tensors={"gate.weight": q + "gate", "up.weight": q + "up", "down.weight": q + "down"})
            layers.append(ParallelLayerSpec("parallel", mixer, feed, self._norm(f"l{i}.norm1")))
        spec = ModelSpec(
            architecture=ARCHITECTURE, embedding=EmbeddingSpec(self.vocab, self.width, {"weight": "embed"}, scale=self.embedding_scale),
            layers=tuple(layers), order=tuple(range(len(layers))), final_norm=self._norm("final.norm"),
            head=HeadSpec(self.vocab, self.width, False, {"weight": "head"}), max_positions=MAX_POSITIONS)
        spec.validate()
        return spec

    # ------------------------------------------------------------------ random weights
    def random_tensor_plan(self):
        """(name, shape, law) of every tensor of a random checkpoint; the laws are those of ``weights.random_init``."""
        w = self.width
        plan = [("embed", (self.vocab, w), "matrix")]
        for i, (m, ff) in enumerate(zip(self.mixers, self.ff)):
            plan += [(f"l{i}.norm1", (w,), "norm"), (f"l{i}.norm1.b", (w,), "bias")]
            p = f"l{i}.mix."
            if isinstance(m, ConvAttentionLayer):
                nq, nk = m.heads * m.dim, m.kv_heads * m.dim
                plan += [(p + "q", (nq, w), "matrix"), (p + "k", (nk, w), "matrix")]
                if m.conv:
                    plan += [(p + "q.conv", (nq, m.conv), "filter"), (p + "k.conv", (nk, m.conv), "filter")]
                plan += [(p + "g", (m.heads, w), "matrix"), (p + "o", (w, nq), "matrix")]
            else:
                plan += [(p + "dq", (m.q_rank, w), "matrix"), (p + "dq.norm", (m.q_rank,), "norm"),
                         (p + "uq", (m.heads * (m.dim + m.rot_dim), m.q_rank), "matrix")]
                if m.kv_from is None:
                    plan += [(p + "dkv", (m.kv_rank + m.rot_dim, w), "matrix"), (p + "dkv.norm", (m.kv_rank,), "norm")]
                plan += [(p + "uk", (m.heads * m.dim, m.kv_rank), "matrix"), (p + "uv", (m.heads * m.vdim, m.kv_rank), "matrix"),
                         (p + "sink", (m.heads,), "bias"), (p + "o", (w, m.heads * m.vdim), "matrix")]
            if ff is not None:
                q = f"l{i}.mlp."
                plan += [(q + "gate", (ff, w), "matrix"), (q + "up", (ff, w), "matrix"), (q + "down", (w, ff), "matrix")]
        plan += [("final.norm", (w,), "norm"), ("final.norm.b", (w,), "bias"), ("head", (self.vocab, w), "matrix")]
        return plan
