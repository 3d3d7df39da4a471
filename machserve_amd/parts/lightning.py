"""Linear attention with a decay per head ("lightning" attention) as a mixer with state of fixed size.

Per step: one product for q, k, v and the gate; per head, token after token in 32-bit,
``S <- decay_h S + silu(k) silu(v)^T`` and ``o = S^T silu(q)``, the ``[dim, vdim]`` state of every head carried in
the request's slot; the heads' outputs normed together (RMS norm with a weight per coordinate), times
``sigmoid(gate)``; the output projection.  Nothing scales the scores but the decay.
"""
from __future__ import annotations

import torch

from .base import Mixer, StateRequest, TensorDecl, require_kernel_sizes
from .registry import register_mixer


@register_mixer("lightning")
class LightningAttention(Mixer):
    graph_safe = True  # reads the requests' rows and slots from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if len(s.decay) != s.heads:
            raise ValueError(f"lightning: {len(s.decay)} decays for {s.heads} heads")
        self.nqk, self.nv = s.heads * s.head_dim, s.heads * s.v_head_dim
        require_kernel_sizes(rt, "lightning", [("hidden size", s.hidden), ("heads x value size", self.nv)])
        limits = getattr(rt.ops, "recurrent_limits", None)
        if limits is not None and s.head_dim > limits()["lightning_dim"]:
            raise ValueError(f"lightning: heads of {s.head_dim}; the kernels take up to {limits()['lightning_dim']}")
        self.decay = torch.tensor([float(v) for v in s.decay], dtype=torch.float32, device=rt.device)
        self.state = None

    def tensor_decls(self):
        s = self.spec
        return [TensorDecl("q.weight", (self.nqk, s.hidden)), TensorDecl("k.weight", (self.nqk, s.hidden)),
                TensorDecl("v.weight", (self.nv, s.hidden)), TensorDecl("g.weight", (self.nv, s.hidden)),
                TensorDecl("o.weight", (s.hidden, self.nv)), TensorDecl("norm.weight", (self.nv,), "vector")]

    def load(self, t):
        self.w_qkvg = torch.cat([t["q.weight"], t["k.weight"], t["v.weight"], t["g.weight"]], dim=0).contiguous()
        self.w_o, self.norm_w = t["o.weight"], t["norm.weight"]

    def cache_request(self):
        s = self.spec
        return StateRequest({"kv": (s.heads, s.head_dim, s.v_head_dim)})

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        qkvg = ops.linear(h, self.w_qkvg)
        # single decoded rows go token after token; portions of prompts in chunks on the matrix cores
        o = ops.lightning_attention(qkvg, s.heads, s.head_dim, s.v_head_dim, self.decay, self.state["kv"], ctx.seq_q_start,
                                    ctx.seq_q_len, ctx.seq_slot, not ctx.decode_only)
        y = ops.gated_rmsnorm(o, qkvg, 2 * self.nqk + self.nv, self.norm_w, s.norm_eps)
        stream.add_linear(y, self.w_o)
