"""Grouped-query attention whose values are its keys, behind a short convolution, over the paged cache.

Per step: q, k and the heads' gate as one product that leaves 32-bit sums; one kernel that finishes a row (causal
convolution over the request's earlier projected rows, of which the last ``taps - 1`` are state of fixed size; unit
norm of every head of q and k; the queries' temperature by position; the sigmoid of the gate) and writes the normed
key and, as the value, the key before its norm into their pages; the framework's paged attention kernels, which also
apply the gate to their output; the output projection.  A head is filled with zeros up to the attention tile's size.
"""
from __future__ import annotations

import torch

from .base import Mixer, PagedKVRequest, StateRequest, TensorDecl, attention_head_size, require_kernel_sizes
from .registry import register_mixer


@register_mixer("conv_attention")
class ConvAttention(Mixer):
    graph_safe = True  # reads positions, rows, slots and addresses from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.kv_heads:
            raise ValueError(f"conv_attention: {s.heads} heads are not a multiple of {s.kv_heads} key/value heads")
        self.nq, self.nk = s.heads * s.head_dim, s.kv_heads * s.head_dim
        self.taps = s.conv_taps or 0  # one tap is a weight per channel and needs no state
        self.hd = attention_head_size(rt, s.head_dim)  # of the pools and of the attention kernels
        require_kernel_sizes(rt, "conv_attention", [("hidden size", s.hidden)], self.hd)
        limits = getattr(rt.ops, "conv_rows_limits", None)
        if limits is not None:
            lim = limits()
            if self.nq + self.nk > lim["row"] or self.taps > lim["taps"]:
                raise ValueError(f"conv_attention: a row of q and k of {self.nq + self.nk} numbers under {self.taps} taps; the kernels "
                                 f"take up to {lim['row']} and {lim['taps']}")
        self.group = self.kpool = self.vpool = self.state = None

    def tensor_decls(self):
        s = self.spec
        decls = [TensorDecl("q.weight", (self.nq, s.hidden)), TensorDecl("k.weight", (self.nk, s.hidden)),
                 TensorDecl("o.weight", (s.hidden, self.nq))]
        if self.taps:
            decls += [TensorDecl("q.conv", (self.nq, self.taps), "vector"), TensorDecl("k.conv", (self.nk, self.taps), "vector")]
        if s.gate:
            decls.append(TensorDecl("g.weight", (s.heads, s.hidden)))
        return decls

    def load(self, t):
        s = self.spec
        parts = [t["q.weight"], t["k.weight"]]
        if s.gate:  # the gate's rows ride in the same product, filled up to a multiple of 8 columns
            g = t["g.weight"]
            fill = -s.heads % 8
            parts += [g] + ([g.new_zeros((fill, s.hidden))] if fill else [])
        self.w_proj = torch.cat(parts, dim=0).contiguous()
        self.conv_w = torch.cat([t["q.conv"], t["k.conv"]], dim=0).contiguous() if self.taps else None
        w_o = t["o.weight"]
        if self.hd != s.head_dim:  # the attention's output has the tile's head size: columns of zeros in between
            w_o = torch.nn.functional.pad(w_o.view(s.hidden, s.heads, s.head_dim), (0, self.hd - s.head_dim)).reshape(s.hidden, -1)
        self.w_o = w_o.contiguous()

    def cache_request(self):
        pages = PagedKVRequest(self.spec.kv_heads, self.hd)
        if self.taps < 2:
            return pages
        return [pages, StateRequest({"conv": (self.taps - 1, self.nq + self.nk)})]

    def bind_cache(self, binding):
        pages = binding[0] if self.taps > 1 else binding
        self.group, self.kpool, self.vpool = pages.group, pages.kpool, pages.vpool
        self.state = binding[1].tensors["conv"] if self.taps > 1 else None

    def attention_rows_per_token(self):
        return self.spec.heads // self.spec.kv_heads

    def attention_rows_per_block(self):
        return self.rt.ops.attention_rows_per_block(self.hd)

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        view = ctx.groups[self.group]
        g = self.attention_rows_per_token()
        proj = ops.linear_split(h, self.w_proj)
        coef, every = s.q_temp if s.q_temp is not None else (0.0, 1)
        q, gate = ops.conv_rows(proj, self.conv_w, self.state, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot, ctx.position_axis(0),
                                s.unit_norm, s.norm_eps, float(coef), int(every), True, s.gate, view.slot_map, self.kpool, self.vpool,
                                s.heads, s.kv_heads, s.head_dim, view.page_size)
        if ctx.decode_only and g <= ops.DECODE_MAX_GROUP:
            o = ops.decode_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_pos0, s.heads, s.kv_heads, self.hd,
                                     view.page_size, None, float(s.scale), None, gate)
        else:
            o = ops.paged_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_pos0,
                                    ctx.attention_work[g], s.heads, s.kv_heads, self.hd, view.page_size, None, float(s.scale),
                                    sinks=None, out_gate=gate)
        stream.add_linear(o, self.w_o)
