"""Nubodra on the GPU: every new kernel alone against the CPU stand-in of the same entry point (written from the
mechanisms' equations) or the plain model's function, and the whole engine (cuts of prompts, decoding, mixed batches with
pages and slots used again, captured steps, generation) against the plain model."""
import pytest
import torch

import nubodra_util as U
from emulated_ops import EmulatedOps
from gpu_util import DEV
from plain import nubodra_plain as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
F32 = 1e-4     # float32 against the plain model in 64-bit


def sharpen_for(dtype):
    """Softmaxes far from flat for the 32-bit runs, where a wrong key must show; milder for bfloat16, whose rounding a
    sharp softmax multiplies."""
    return 8.0 if dtype == torch.float32 else 3.0


def ops_of(dtype):
    from machserve_amd.kernels import get_ops
    return get_ops(dtype, DEV)


def dev(t, dtype=None):
    return t.to(device=DEV, dtype=dtype or t.dtype).contiguous()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def close(got, want, dtype, what="", scale_by=None):
    got, want = got.float().cpu().double(), want.double().cpu()
    bound = (1e-4 if dtype == torch.float32 else 2e-2) * float((scale_by if scale_by is not None else want).abs().max()) + 1e-6
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: error {err:.3e} over {bound:.3e}"


# ------------------------------------------------------------------ kernels, each alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [48, 200, 1030])
def test_layer_norm_with_pending_sums_and_gathered_rows(dtype, d):
    ops = ops_of(dtype)
    torch.manual_seed(d)
    x, w, b = torch.randn(7, d) * 2 + 0.5, torch.randn(d), torch.randn(d)
    pend = torch.randn(3, 7, d)
    want = P.layer_norm((x + pend.sum(0)).double(), w.double(), b.double(), 1e-5)
    xs = dev(x)
    got = ops.layernorm(xs, dev(w), dev(b), 1e-5, None, False, dev(pend))
    close(got, want, dtype, "layer norm over pending sums")
    close(xs, x + pend.sum(0), torch.float32, "the stream took the pending sums")
    rows = [5, 0, 5]
    got = ops.layernorm(dev(x), dev(w), None, 1e-5, i32(rows), True, None)
    close(got, P.layer_norm(x.double(), w.double(), torch.zeros(d, dtype=torch.float64), 1e-5)[rows], torch.float32, "gathered rows, no bias")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,B,N,K", [(1, 3, 24, 16), (5, 6, 26, 32), (16, 2, 300, 40), (17, 4, 64, 96), (200, 5, 80, 136), (70, 20, 40, 8)])
def test_product_per_head(dtype, T, B, N, K):
    ops = ops_of(dtype)
    torch.manual_seed(T + N)
    a, w = torch.randn(T, B, K), torch.randn(B, N, K)
    want = torch.einsum("tbk,bnk->tbn", a.to(dtype).double(), w.to(dtype).double())
    close(ops.heads_linear(dev(a, dtype), dev(w, dtype)), want, dtype, "a new output")
    out = torch.full((T, B, N + 5), 7.0, dtype=dtype, device=DEV)
    ops.heads_linear(dev(a, dtype), dev(w, dtype), out)
    close(out[..., :N], want, dtype, "into the first columns of wider heads")
    assert bool((out[..., N:] == 7.0).all()), "the columns behind were written"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank,rank,rot,hd,own", [(40, 24, 8, 32, True), (20, 26, 6, 32, True), (9, 26, 6, 32, False), (96, 60, 20, 80, True),
                                                     (16, 12, 0, 16, True)])
def test_rows_of_the_latent_and_its_queries(dtype, q_rank, rank, rot, hd, own):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(q_rank)
    T, ps, H, d = 9, 16, 3, 12
    n = q_rank + (rank + rot if own else 0)
    proj = torch.randn(2, T, n + 3)
    qn, cn = torch.rand(q_rank) + 0.5, torch.rand(rank) + 0.5
    inv_freq = torch.rand(max(rot // 2, 1))[:rot // 2]
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 1000, 7, 8], dtype=torch.int32)
    slot_map = torch.tensor([16, 17, 18, 19, 40, 41, 63, 0, 1], dtype=torch.int32)
    pools = lambda: (torch.zeros(4, 1, ps, hd, dtype=dtype), torch.zeros(4, 1, hd, ps, dtype=dtype))
    (k0, v0), (k1, v1) = pools(), pools()
    k1, v1 = dev(k1), dev(v1)
    want = ref.latent_rows(proj, qn, cn if own else None, 1e-5, pos, inv_freq if rot else None, 1.3, slot_map, k0, v0, q_rank, rank, rot, ps)
    got = ops.latent_rows(dev(proj), dev(qn), dev(cn) if own else None, 1e-5, dev(pos), dev(inv_freq) if rot and own else None, 1.3,
                          dev(slot_map) if own else None, k1 if own else None, v1 if own else None, q_rank, rank, rot, ps)
    close(got, want, dtype, "query latent")
    assert got.shape[1] % 8 == 0 and bool((got[:, q_rank:] == 0).all())
    if own:
        close(k1, k0, dtype, "keys: latent, rotated part, zeros behind")
        close(v1, v0, dtype, "values: the latent")
        assert bool((k1[..., rank + rot:] == 0).all()) and bool((v1[:, :, rank:] == 0).all())
    q = torch.randn(T, H * (d + rot))
    plain_w, att_w = ref.latent_query(q, pos, inv_freq if rot else None, 1.3, H, d, rot, rank, hd)
    plain_g, att_g = ops.latent_query(dev(q), dev(pos), dev(inv_freq) if rot else None, 1.3, H, d, rot, rank, hd)
    close(plain_g, plain_w, dtype, "plain parts of the queries")
    close(att_g[..., rank:], att_w[..., rank:], dtype, "rotated parts behind the latent's columns")


def test_rotation_of_the_latent_kernels_is_the_plain_models():
    ops = ops_of(torch.float32)
    rot = {"base": 300.0, "dims": 6, "scaling": {"factor": 3.0, "original": 32, "fast": 6.0, "slow": 1.0}}
    f, factor = P.rotary_frequencies(rot)
    pos = torch.tensor([0, 3, 77], dtype=torch.int32)
    q = torch.randn(3, 2 * (4 + 6))
    _, att = ops.latent_query(dev(q), dev(pos), dev(f.float()), factor, 2, 4, 6, 8, 16)
    want = P.rotate_interleaved(q.view(3, 2, 10)[..., 4:].double(), pos, rot)
    close(att[..., 8:14], want, torch.float32, "neighbouring pairs, scaled frequencies, factor on cosines and sines")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,taps,temp", [(4, 2, 24, 4, (0.7, 5)), (6, 1, 20, 5, (1.5, 7)), (3, 3, 16, 2, (0.2, 1)), (2, 2, 8, 0, None), (2, 2, 8, 1, None),
                                              (18, 1, 16, 3, (0.5, 16)), (2, 1, 72, 7, (0.3, 128)), (2, 1, 24, 9, (0.3, 4)), (1, 1, 136, 8, None)])
@pytest.mark.parametrize("lens", [[11, 1, 6], [75, 1, 40]])
def test_rows_behind_the_convolution_in_one_step_and_in_many(dtype, H, KV, d, taps, temp, lens):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(H * d + taps)
    ps, hd = 128, -(-d // 16) * 16  # a page a request
    C = (H + KV) * d
    T = sum(lens)
    proj = torch.randn(2, T, C + -(-H // 8) * 8)
    conv_w = torch.randn(C, taps) * 0.5 if taps else None
    coef, every = temp or (0.0, 1)

    def run(o, cuts, to):
        """The three requests' rows in steps of the given sizes (a request's share of a step: its next `cut` rows)."""
        state = to(torch.zeros(5, taps - 1, C)) if taps > 1 else None
        kp, vp = to(torch.zeros(6, KV, ps, hd, dtype=dtype)), to(torch.zeros(6, KV, hd, ps, dtype=dtype))
        qs, gates = [None] * T, [None] * T
        starts = [0, lens[0], lens[0] + lens[1]]
        at = [0, 0, 0]
        while any(a < n for a, n in zip(at, lens)):
            rows, q0, ql, slots = [], [], [], []
            for s in range(3):
                c = min(cuts[s], lens[s] - at[s])
                if c > 0:
                    q0.append(len(rows)); ql.append(c); slots.append(s + 1)
                    rows += list(range(starts[s] + at[s], starts[s] + at[s] + c))
                    at[s] += c
            pos = [r - starts[max(i for i in range(3) if starts[i] <= r)] for r in rows]
            slot_map = [(1 + max(i for i in range(3) if starts[i] <= r)) * ps + p for r, p in zip(rows, pos)]  # a page a request
            it = lambda v: to(torch.tensor(v, dtype=torch.int32))
            q, g = o.conv_rows(to(proj[:, rows].contiguous()), to(conv_w) if taps else None, state, it(q0), it(ql), it(slots), it(pos), True, 1e-5,
                               coef, every, True, True, it(slot_map), kp, vp, H, KV, d, ps)
            for i, r in enumerate(rows):
                qs[r], gates[r] = q[i].float().cpu(), g[i].float().cpu()
        return torch.stack(qs), torch.stack(gates), kp.float().cpu(), vp.float().cpu(), None if state is None else state.float().cpu()

    want = run(ref, [100, 100, 100], lambda t: t.clone())
    for cuts in ([100, 100, 100], [1, 1, 1], [2, 1, 5], [3, 1, 1], [64, 1, 29]):
        got = run(ops, cuts, lambda t: dev(t))
        for g, w, what in zip(got, want, ("queries", "gates", "keys", "values", "state")):
            if w is not None:
                close(g, w, dtype, f"{what}, steps of {cuts}")
    # the plain model's mechanisms on the first request, whole
    row = proj.sum(0)[:lens[0], :C].double()
    y = P.causal_conv(row, conv_w.double()) if taps else row
    q, k = y[:, :H * d].view(-1, H, d), y[:, H * d:].view(-1, KV, d)
    qn = P.rms(q, 1e-5) * P.query_temperature(lens[0], coef, every, torch.float64)[:, None, None] if temp else P.rms(q, 1e-5)
    close(want[0][:lens[0]].view(-1, H, hd)[..., :d], qn, dtype, "queries against the plain mechanisms")
    close(want[2][1, :, :lens[0], :d].transpose(0, 1), P.rms(k, 1e-5), dtype, "keys against the plain mechanisms")
    close(want[3][1, :, :d, :lens[0]].permute(2, 0, 1), k, dtype, "values are the keys before their norm")


def _attention_case(dtype, H, KV, hd, ps, before, now, seed, sinks, gated, spike=None, key_splits=0):
    """Requests with ``before[i]`` keys in the cache and ``now[i]`` rows in the step; kernel against stand-in."""
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(seed)
    S, T = len(now), sum(now)
    total = [b + n for b, n in zip(before, now)]
    width = max(-(-t // ps) for t in total)
    pages = sum(-(-t // ps) for t in total) + 1
    perm = torch.randperm(pages - 1) + 1
    table, at = torch.full((S, width), -1, dtype=torch.int32), 0
    for s, t in enumerate(total):
        n = -(-t // ps)
        table[s, :n] = perm[at:at + n].int()
        at += n
    kpool, vpool = torch.randn(pages, KV, ps, hd).to(dtype), torch.randn(pages, KV, hd, ps).to(dtype)
    q = torch.randn(T, H * hd)
    if spike is not None:   # one (request, key) whose score stands out for every head of the request's last row
        s, key = spike
        page, off = int(table[s, key // ps]), key % ps
        row = sum(now[:s + 1]) - 1
        for h in range(H):
            kpool[page, h // (H // KV), off] = (q[row, h * hd:(h + 1) * hd] * 4).to(dtype) if h % (H // KV) == 0 else kpool[page, h // (H // KV), off]
        vpool[page, :, :, off] = 50.0
    q = q.to(dtype)
    sk = torch.randn(H) * 2 if sinks else None
    gate = torch.rand(T, H) if gated else None
    q0 = torch.tensor([sum(now[:s]) for s in range(S)], dtype=torch.int32)
    ql, p0 = torch.tensor(now, dtype=torch.int32), torch.tensor(before, dtype=torch.int32)
    g = H // KV
    unit = ops.attention_rows_per_block(hd)
    ref.rows_per_block = unit
    work = torch.tensor([[s, r0] for s in range(S) for r0 in range(0, now[s] * g, unit)], dtype=torch.int32)
    scale = 0.2
    want = ref.paged_attention(q, kpool, vpool, table, q0, ql, p0, work, H, KV, hd, ps, None, scale, sinks=sk, out_gate=gate)
    opt = lambda t: None if t is None else dev(t)
    got = ops.paged_attention(dev(q), dev(kpool), dev(vpool), dev(table), dev(q0), dev(ql), dev(p0), dev(work), H, KV, hd, ps, None, scale,
                              key_splits=key_splits, sinks=opt(sk), out_gate=opt(gate))
    close(got, want, dtype, f"mixed-batch kernel ({key_splits} splits)", scale_by=want.abs().max().clamp(min=1.0))
    if all(n == 1 for n in now) and g <= ops.DECODE_MAX_GROUP:
        got = ops.decode_attention(dev(q), dev(kpool), dev(vpool), dev(table), dev(p0), H, KV, hd, ps, None, scale, opt(sk), opt(gate))
        close(got, want, dtype, "decode kernel", scale_by=want.abs().max().clamp(min=1.0))
    return want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sinks,gated", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("H,KV,hd", [(6, 1, 80), (4, 2, 48), (20, 1, 32), (8, 8, 64), (16, 1, 256)])
def test_attention_with_a_sink_and_an_output_gate(dtype, sinks, gated, H, KV, hd):
    _attention_case(dtype, H, KV, hd, 16, [0, 5, 130], [40, 1, 9], 1, sinks, gated)
    _attention_case(dtype, H, KV, hd, 16, [0, 5, 130], [40, 1, 9], 2, sinks, gated, key_splits=3)
    _attention_case(dtype, H, KV, hd, 16, [600, 17, 0, 255], [1, 1, 1, 1], 3, sinks, gated)          # decoding; the long one in splits
    _attention_case(dtype, H, KV, hd, 64, [1000], [1], 4, sinks, gated)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("key", [0, 15, 16, 63, 64, 400, 798, 799])
def test_a_key_that_stands_out_is_seen_wherever_it_lies(dtype, decoded, key):
    """The first key, the last of a page and the first of the next, a key hundreds back, the row's neighbour and the row
    itself: the spiked key takes all the weight beside the sink, so its value (50 in every column) is what comes out."""
    n = 800
    want = _attention_case(dtype, 6, 1, 80, 16, [n - 1] if decoded else [0], [1] if decoded else [n], 5, True, False, spike=(0, key))
    assert float(want[-1, :80].min()) > 25.0


def test_a_sink_far_above_the_scores_takes_the_weight():
    ops = ops_of(torch.float32)
    H, hd, ps = 2, 16, 16
    kpool, vpool = torch.randn(2, 1, ps, hd), torch.ones(2, 1, hd, ps)
    q = torch.randn(1, H * hd)
    table = i32([[1]])
    sink = torch.tensor([40.0, -40.0])
    got = ops.decode_attention(dev(q), dev(kpool), dev(vpool), table, i32([3]), H, 1, hd, ps, None, 0.1, dev(sink), None).cpu()
    assert float(got[0, :hd].abs().max()) < 1e-6 and abs(float(got[0, hd]) - 1.0) < 1e-5


# ------------------------------------------------------------------ the engine
def loaded(model_dir, dtype, page_size=16, max_tokens=1024, max_requests=4, use_graphs=True, num_pages=None):
    from machserve_amd.engine.loading import load_model
    return load_model(model_dir, dtype=dtype, device=DEV, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests,
                      use_graphs=use_graphs, num_pages=num_pages)


def _cut(rid, n, sizes):
    out, at, k = [], 0, 0
    while at < n:
        c = min(sizes[k % len(sizes)], n - at)
        out.append([(rid, c)])
        at, k = at + c, k + 1
    return out


def plain_for(model_dir, dtype, tokens):
    """The plain model in 64-bit, on the weights as the run holds them."""
    return U.plain_logits(model_dir, tokens, torch.float64, weights_as=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_prompts_cut_anywhere_and_decoding_equal_the_plain_model(tmp_path, name, dtype):
    d = U.make_dir(tmp_path, name, seed=7, sharpen=sharpen_for(dtype))
    n = 150
    toks = U.tokens_of(n, U.CONFIGS[name]["vocab"], 8)
    want = plain_for(d, dtype, toks)
    lm = loaded(d, dtype)
    schedules = {"whole": [[("a", n)]], "prompt, then token by token": [[("a", 60)]] + [[("a", 1)]] * (n - 60),
                 "portions down to two tokens": _cut("a", n, [2, 33, 3, 16, 2, 47, 1, 1, 31, 2])}
    for what, schedule in schedules.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.within(got, want, dtype), what
    lm.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [False, True])
def test_unequal_requests_side_by_side_equal_each_alone(tmp_path, dtype, graphs):
    name = "pair"
    d = U.make_dir(tmp_path, name, seed=9, sharpen=sharpen_for(dtype))
    vocab = U.CONFIGS[name]["vocab"]
    reqs = {"a": U.tokens_of(90, vocab, 1), "b": U.tokens_of(1, vocab, 2), "c": U.tokens_of(41, vocab, 3),
            "d": U.tokens_of(70, vocab, 4), "e": U.tokens_of(35, vocab, 5)}
    schedule = [[("b", 1), ("a", 20), ("c", 5)], [("a", 1), ("c", 30)], [("a", 2), ("c", 2), ("d", 17)], [("a", 1), ("c", 1), ("d", 1)],
                [("a", 1), ("c", 1), ("d", 1)], [("a", 1), ("c", 1), ("d", 1)], [("a", 1), ("c", 1), ("d", 1)],
                [("d", 1), ("e", 16), ("a", 1)], [("a", 30), ("e", 1), ("d", 2)], [("a", 32), ("d", 46), ("e", 18)]]
    lm = loaded(d, dtype, max_requests=3, num_pages=16, use_graphs=graphs)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.within(got[i], plain_for(d, dtype, toks), dtype), i
    if dtype == torch.float32:      # and the same numbers, beyond rounding, as each request alone in one step
        alone = loaded(d, dtype, use_graphs=False)
        for i, toks in reqs.items():
            assert U.relative_error(got[i], U.run_schedule(alone, {i: toks}, [[(i, len(toks))]])[i]) < 1e-5, i
    lm.cache.check()
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["odd", "heads"])
def test_long_decoding_from_captured_steps(tmp_path, name, dtype):
    d = U.make_dir(tmp_path, name, seed=10, sharpen=sharpen_for(dtype))
    toks = U.tokens_of(330, U.CONFIGS[name]["vocab"], 3)
    lm = loaded(d, dtype, max_tokens=512)
    got = U.run_schedule(lm, {"a": toks}, [[("a", 10)]] + [[("a", 1)]] * 320)["a"]
    assert U.within(got, plain_for(d, dtype, toks), dtype)
    assert len(lm.step._graphs) > 0     # the single rows ran from captured steps


def test_a_long_prompt_in_portions_behind_pages_of_64(tmp_path):
    """Keys far away and across many pages, in a step of many rows and in portions that end inside pages."""
    d = U.make_dir(tmp_path, "pair", seed=11)
    toks = U.tokens_of(1100, 97, 6)
    want = plain_for(d, torch.float32, toks)
    lm = loaded(d, torch.float32, page_size=64, max_tokens=1152)
    for what, schedule in {"whole": [[("a", 1100)]], "portions": _cut("a", 1100, [500, 63, 2, 129, 300, 7])}.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.relative_error(got, want) < F32, what


def test_first_tokens_of_a_sequence(tmp_path):
    for name in sorted(U.CONFIGS):
        d = U.make_dir(tmp_path, name, seed=12)
        toks = U.tokens_of(4, U.CONFIGS[name]["vocab"], 1)
        lm = loaded(d, torch.float32)
        for n in (1, 2, 3, 4):
            got = U.run_schedule(lm, {"a": toks[:n]}, [[("a", n)]])["a"]
            assert U.relative_error(got, plain_for(d, torch.float32, toks[:n])) < F32, (name, n)
            got = U.run_schedule(lm, {"a": toks[:n]}, [[("a", 1)]] * n)["a"]
            assert U.relative_error(got, plain_for(d, torch.float32, toks[:n])) < F32, (name, n, "one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, dtype):
    import machserve_amd
    d = U.make_dir(tmp_path, "pair", seed=13, sharpen=3.0)
    w, cfg = U.read(d)
    prompts = [U.tokens_of(n, 97, n) for n in (3, 21, 1, 40, 17)]
    got = machserve_amd.generate(d, prompts, max_new=8, dtype=dtype, page_size=16, capacity=3, max_batch_tokens=32, chunk_size=16)
    for p, g in zip(prompts, got):
        if dtype == "float32":
            assert g == P.greedy_generate(w, cfg, p, 8, torch.float64)
        else:   # bfloat16 may flip a near-tie: every token must be within rounding of the best
            seq = list(p)
            for t in g:
                logits = plain_for(d, torch.bfloat16, seq)[-1]
                assert logits[t] >= logits.max() - 5e-2 * (logits.max() - logits.min()), "a token that is not a maximum"
                seq.append(t)


def test_a_folder_of_this_layout_runs_through_the_trace_program(tmp_path):
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    d = U.make_dir(tmp_path, "odd", seed=14)
    toks = U.tokens_of(50, 61, 2)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[33:], "want": [16]}, {"id": "y", "tokens": toks[:2], "want": []}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128", "--page-size", "16"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1"]
    want = plain_for(d, torch.float32, toks)
    got = torch.from_numpy(np.concatenate([np.fromfile(out / "0.f32", dtype="<f4"), np.fromfile(out / "1.f32", dtype="<f4")]).reshape(3, 61))
    assert U.relative_error(got, want[[0, 32, 49]]) < F32


def test_command_line_generates_from_a_folder(tmp_path):
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    d = U.make_dir(tmp_path, "pair", seed=15)
    w, cfg = U.read(d)
    prompt = U.tokens_of(9, 97, 4)
    cmd = [sys.executable, os.path.join(root, "bin", "machserve"), "--max-new", "5", "--dtype", "f32", "--tpp", "16", "--prompt-ids"]
    r = subprocess.run(cmd + [",".join(map(str, prompt)), "--model", d], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.split()] == P.greedy_generate(w, cfg, prompt, 5, torch.float64)
