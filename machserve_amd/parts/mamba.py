"""The Mamba layer (selective scan) as a mixer with state of fixed size.

Per step: the input projection to ``[x | z]``; a causal convolution per channel with SiLU, whose last
``taps - 1`` inputs of every request are state; a projection of the convolved ``x`` to the step sizes' input, B
and C; the scan ``S <- exp(dt A) S + dt x B``, ``y = S . C + D x`` with ``dt = softplus(W_dt low + b)`` and
``A = -exp(A_log)``, token after token in 32-bit, the ``[channels, states]`` state carried in the request's slot;
the gate ``y * silu(z)``; the output projection.
"""
from __future__ import annotations

from .base import Mixer, StateRequest, TensorDecl, require_kernel_sizes
from .registry import register_mixer


@register_mixer("mamba1")
class SelectiveScan(Mixer):
    graph_safe = True  # reads the requests' rows and slots from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        require_kernel_sizes(rt, "mamba1", [("hidden size", spec.hidden), ("inner size", spec.inner)])
        limits = getattr(rt.ops, "recurrent_limits", None)
        if limits is not None:
            lim = limits()
            if spec.conv_taps > lim["taps"] or spec.states > lim["states"]:
                raise ValueError(f"mamba1: {spec.conv_taps} taps and {spec.states} states a channel; the kernels take up to "
                                 f"{lim['taps']} and {lim['states']}")
        self.state = None

    def tensor_decls(self):
        s = self.spec
        return [TensorDecl("in.weight", (2 * s.inner, s.hidden)), TensorDecl("conv.weight", (s.inner, s.conv_taps), "vector"),
                TensorDecl("conv.bias", (s.inner,), "vector"), TensorDecl("x.weight", (s.dt_rank + 2 * s.states, s.inner)),
                TensorDecl("dt.weight", (s.inner, s.dt_rank), "vector"), TensorDecl("dt.bias", (s.inner,), "vector"),
                TensorDecl("A_log", (s.inner, s.states), "vector"), TensorDecl("D", (s.inner,), "vector"),
                TensorDecl("o.weight", (s.hidden, s.inner))]

    def load(self, t):
        self.w_in, self.w_x, self.w_o = t["in.weight"], t["x.weight"], t["o.weight"]
        self.conv_w, self.conv_b = t["conv.weight"], t["conv.bias"]
        # the step sizes' projection is kept transposed, [dt_rank, channels]: the kernel's threads are channels
        self.w_dt = t["dt.weight"].t().contiguous()
        self.b_dt, self.a_log, self.d_skip = t["dt.bias"], t["A_log"], t["D"]

    def cache_request(self):
        s = self.spec
        return StateRequest({"conv": (max(s.conv_taps - 1, 1), s.inner), "scan": (s.inner, s.states)})

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        seqs = (ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        xz = ops.linear(h, self.w_in)
        x = ops.causal_conv(xz, s.inner, self.conv_w, self.conv_b, self.state["conv"], *seqs)
        dbc = ops.linear(x, self.w_x, None, out_f32=True)
        y = ops.selective_scan(x, xz, dbc, s.dt_rank, s.states, self.w_dt, self.b_dt, self.a_log, self.d_skip, self.state["scan"], *seqs)
        stream.add_linear(y, self.w_o)
