"""Grouped-query attention whose heads exchange their scores before the softmax, over the paged cache.

Per step: the q/k/v projection as one product that leaves 32-bit sums; one kernel that finishes a row (RMS norm
over the whole query and the whole key projection, rotation of the first part of every head, values blended with
those the first such layer computed for the same token) and writes key and value into their pages; one kernel for
the attention of every row over the keys it sees (the last ``window`` positions and the request's first
``keep_first``), in which the scaled scores of all heads for a key are mixed by a square matrix before each head's
softmax; the output projection.  Keys are ``head_dim`` wide, values ``v_head_dim``.
"""
from __future__ import annotations

import torch

from .base import Mixer, PagedKVRequest, PendingNorm, TensorDecl, require_kernel_sizes
from .registry import POSITION_ENCODINGS, register_mixer


@register_mixer("talking_attention")
class TalkingAttention(Mixer):
    graph_safe = True          # reads positions and addresses from device memory only
    takes_pending_norm = True  # its first product can apply the norm of the stream itself

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.kv_heads:
            raise ValueError(f"talking_attention: {s.heads} heads are not a multiple of {s.kv_heads} key/value heads")
        if s.value_blend not in (None, "source", "blend"):
            raise ValueError(f"talking_attention: value_blend {s.value_blend!r} is none of None, 'source', 'blend'")
        self.nq, self.nk, self.nv = s.heads * s.head_dim, s.kv_heads * s.head_dim, s.kv_heads * s.v_head_dim
        require_kernel_sizes(rt, "talking_attention", [("hidden size", s.hidden), ("heads x value size", s.heads * s.v_head_dim)])
        limits = getattr(rt.ops, "talking_limits", None)
        if limits is not None and self.nq + self.nk + self.nv > limits()["row"]:
            raise ValueError(f"talking_attention: a row of q, k and v of {self.nq + self.nk + self.nv} numbers exceeds the kernels' "
                             f"{limits()['row']}")
        self.position = POSITION_ENCODINGS.build(s.position, rt) if s.position is not None else None
        self.group = self.kpool = self.vpool = None

    def sub_parts(self):
        return [self.position] if self.position is not None else []

    def tensor_decls(self):
        s = self.spec
        decls = [TensorDecl("q.weight", (self.nq, s.hidden)), TensorDecl("k.weight", (self.nk, s.hidden)),
                 TensorDecl("v.weight", (self.nv, s.hidden)), TensorDecl("o.weight", (s.hidden, s.heads * s.v_head_dim))]
        if s.qk_norm:
            decls += [TensorDecl("q_norm.weight", (self.nq,), "vector"), TensorDecl("k_norm.weight", (self.nk,), "vector")]
        if s.talk:
            decls.append(TensorDecl("talk", (s.heads, s.heads), "vector"))
        if s.value_blend == "blend":
            decls.append(TensorDecl("blend", (), "vector"))
        return decls

    def ignored_tensors(self):
        """A layer that does not blend (the one whose values the others blend with, or one outside the blending) may
        have a blend weight in the checkpoint that nothing reads."""
        return [self.spec.tensors.get("blend", "blend")] if self.spec.value_blend != "blend" else []

    def load(self, t):
        self.w_qkv = torch.cat([t["q.weight"], t["k.weight"], t["v.weight"]], dim=0).contiguous()
        self.w_o = t["o.weight"]
        self.q_norm, self.k_norm = t.get("q_norm.weight"), t.get("k_norm.weight")
        self.talk = t.get("talk")
        self.blend = t["blend"].reshape(1).contiguous() if self.spec.value_blend == "blend" else None

    def cache_request(self):
        s = self.spec
        return PagedKVRequest(s.kv_heads, s.head_dim, s.window, s.v_head_dim, s.keep_first if s.window else 0)

    def bind_cache(self, binding):
        self.group, self.kpool, self.vpool = binding.group, binding.kpool, binding.vpool

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        view = ctx.groups[self.group]
        qkv = h.linear_split(self.w_qkv) if isinstance(h, PendingNorm) else ops.linear_split(h, self.w_qkv)
        pos = self.position
        shared = ("values of the first blending layer", s.kv_heads, s.v_head_dim)
        other = None
        if s.value_blend == "blend":
            other = ctx.shared.get(shared)
            if other is None:
                raise ValueError("talking_attention: a layer blends its values, but no layer before it has kept its own")
        q, own = ops.talking_prepare(qkv, self.q_norm, self.k_norm, s.norm_eps, ctx.position_axis(0),
                                     pos.inv_freq if pos is not None else None, pos.rotary_dim if pos is not None else 0,
                                     pos.factor if pos is not None else 1.0, other, self.blend, s.value_blend == "source",
                                     view.slot_map, self.kpool, self.vpool, s.heads, s.kv_heads, s.head_dim, s.v_head_dim,
                                     view.page_size)
        if s.value_blend == "source":
            ctx.shared[shared] = own
        # a step of many rows a request runs in tiles of 16 rows on the matrix cores, single decoded rows (and steps that
        # are mostly such rows: a tile takes its requests one after the other) one row a block
        tiles = not ctx.decode_only and ctx.n_rows >= max(getattr(ops, "TILE_MIN_ROWS", 1 << 30), 4 * ctx.n_seqs)
        o = ops.talking_attention(q, self.kpool, self.vpool, self.talk, view.block_table, ctx.seq_q_start, ctx.seq_pos0, s.heads,
                                  s.kv_heads, s.head_dim, s.v_head_dim, view.page_size, s.window, s.keep_first, float(s.scale),
                                  ctx.seq_q_len, tiles)
        stream.add_linear(o, self.w_o)
