"""Renanex on the GPU: every kernel of its mixers against the plain model's function of the same mechanism, and the whole
engine (cuts of prompts, decoding, mixed batches, captured steps, generation) against the plain model."""
import math

import pytest
import torch

import renanex_util as U
from gpu_util import DEV
from plain import renanex_plain as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
F32 = 1e-4     # float32 against the plain model in 64-bit, as renanex_util.within allows it


def sharpen_for(dtype):
    """Softmaxes far from flat for the 32-bit runs, where a wrong key must show; as drawn for bfloat16, whose rounding a
    sharp softmax would multiply."""
    return 2.0 if dtype == torch.float32 else 1.0


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
def test_norm_add_and_softcap(dtype):
    ops = ops_of(dtype)
    torch.manual_seed(0)
    for rows, width, sums in ((5, 72, 3), (3, 70, 1), (17, 2048, 19)):   # four columns a thread, or one where the width is odd
        x, parts, w = torch.randn(rows, width), torch.randn(sums, rows, width), torch.randn(width)
        y = parts.double().sum(0)
        want = x.double() + P.rms(y, 1e-5) * w.double()
        xd = dev(x)
        ops.norm_add(xd, dev(parts), dev(w), 1e-5)
        close(xd, want, torch.float32, f"norm_add of {sums} sums of width {width}")
    logits = torch.randn(4, 333) * 20
    ld = dev(logits)
    ops.softcap(ld, 0.25, 7.0)
    close(ld, 7.0 * torch.tanh(logits.double() * 0.25 / 7.0), torch.float32, "softcap")
    ld = dev(logits)
    ops.softcap(ld, 0.5, 0.0)
    close(ld, logits.double() * 0.5, torch.float32, "scale without a cap")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_causal_convolution_carries_its_last_inputs(dtype, taps):
    ops = ops_of(dtype)
    torch.manual_seed(taps)
    C, lens = 40, [9, 1, 3]
    w, b = torch.randn(C, taps), torch.randn(C)
    total = {s: torch.randn(n + 5, 2 * C).to(dtype).float() for s, n in enumerate(lens)}   # a first step of n rows, then 1 + 4
    state = torch.zeros(5, max(taps - 1, 1), C, device=DEV)
    slots = [3, 0, 2]
    got = {s: [] for s in total}
    for step in range(3):
        counts = [lens[s] if step == 0 else (1 if step == 1 else 4) for s in range(3)]
        first = [0 if step == 0 else (lens[s] if step == 1 else lens[s] + 1) for s in range(3)]
        rows = torch.cat([total[s][first[s]:first[s] + counts[s]] for s in range(3)])
        starts = [sum(counts[:s]) for s in range(3)]
        out = ops.causal_conv(dev(rows, dtype), C, dev(w), dev(b), state, i32(starts), i32(counts), i32(slots))
        for s in range(3):
            got[s].append(out[starts[s]:starts[s] + counts[s]].float().cpu())
    for s, x in total.items():
        padded = torch.cat([torch.zeros(taps - 1, C), x[:, :C]]).double()
        want = sum(padded[k:k + x.shape[0]] * w[:, k].double() for k in range(taps)) + b.double()
        close(torch.cat(got[s]), P.silu(want), dtype, f"convolution of request {s}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,N,R", [(24, 3, 1), (70, 16, 5), (40, 24, 12), (33, 40, 2)])
def test_selective_scan_in_one_step_and_in_many(dtype, C, N, R):
    ops = ops_of(dtype)
    torch.manual_seed(C)
    n = 37
    x, z = (torch.randn(n, C).to(dtype).float() for _ in range(2))
    dbc = torch.randn(n, R + 2 * N)
    w_dt, b_dt, a_log, dsk = torch.randn(C, R) * 0.5, torch.randn(C) - 2.0, torch.randn(C, N) * 0.5, torch.randn(C)
    dt = P.softplus(dbc[:, :R].double() @ w_dt.double().T + b_dt.double())
    A = -torch.exp(a_log.double())
    S, want = torch.zeros(C, N, dtype=torch.float64), torch.empty(n, C, dtype=torch.float64)
    for i in range(n):
        S = torch.exp(dt[i][:, None] * A) * S + (dt[i] * x[i].double())[:, None] * dbc[i, R:R + N].double()[None, :]
        want[i] = S @ dbc[i, R + N:].double() + dsk.double() * x[i].double()
    want = want * P.silu(z.double())
    xz = torch.cat([torch.zeros(n, C), z], 1)
    for cuts in ([n], [1] * n, [5, 2, 29, 1]):
        state = torch.zeros(3, C, N, device=DEV)
        state[0] = 7.0   # another request's: must stay
        got, at = [], 0
        for c in cuts:
            got.append(ops.selective_scan(dev(x[at:at + c], dtype), dev(xz[at:at + c], dtype), dev(dbc[at:at + c]), R, N, dev(w_dt.t()),
                                          dev(b_dt), dev(a_log), dev(dsk), state, i32([0]), i32([c]), i32([1])))
            at += c
        close(torch.cat(got), want, dtype, f"scan cut as {cuts[:4]}")
        close(state[1], S, torch.float32, "the state after the last token")
        assert float(state[0].min()) == 7.0 and float(state[2].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_lightning_attention_in_segments_equals_the_walk_token_after_token(dtype):
    """Steps of many rows cut their requests into segments that are walked side by side."""
    ops = ops_of(dtype)
    torch.manual_seed(6)
    H, d, dv, lens = 2, 24, 40, [300, 129, 1, 260]
    T, seg = sum(lens), ops.LIGHTNING_SEGMENT
    assert T >= 2 * seg and T // len(lens) >= seg
    rows = (torch.randn(T, 2 * H * d + 2 * H * dv) * 0.5).to(dtype).float()
    decay = torch.tensor([0.9, 0.995])
    start = torch.randn(6, H, d, dv)
    slots, starts = [4, 0, 2, 5], [0, 300, 429, 430]
    state = dev(start.clone())
    got = ops.lightning_attention(dev(rows, dtype), H, d, dv, dev(decay), state, i32(starts), i32(lens), i32(slots), True)
    for s, (q0, n) in enumerate(zip(starts, lens)):     # each request alone, token after token
        alone = dev(start.clone())
        want = torch.cat([ops.lightning_attention(dev(rows[t:t + 1], dtype), H, d, dv, dev(decay), alone, i32([0]), i32([1]), i32([slots[s]]))
                          for t in range(q0, q0 + n)])
        close(got[q0:q0 + n], want, dtype, f"request {s} in segments")
        close(state[slots[s]], alone[slots[s]], dtype, f"state of request {s}")
    assert torch.equal(state[1].cpu(), start[1]) and torch.equal(state[3].cpu(), start[3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,N", [(48, 12), (70, 24), (33, 40)])
def test_a_long_scan_in_chunks_equals_the_walk_token_after_token(dtype, C, N):
    """Steps of many rows cut their requests into chunks that are walked side by side; the result is the one walk's."""
    ops = ops_of(dtype)
    torch.manual_seed(5)
    R, lens = 3, [300, 1, 129, 210]
    T = sum(lens)
    assert T >= ops.SCAN_CHUNK_MIN_ROWS and T // len(lens) >= ops.SCAN_CHUNK_MIN_ROWS // 2
    x, z = (torch.randn(T, C).to(dtype).float() for _ in range(2))
    dbc = torch.randn(T, R + 2 * N)
    w_dt, b_dt, a_log, dsk = torch.randn(C, R) * 0.5, torch.randn(C) - 2.0, torch.randn(C, N) * 0.5, torch.randn(C)
    start = torch.randn(6, C, N)
    slots, starts = [4, 0, 2, 5], [0, 300, 301, 430]
    args = lambda rows: (dev(x[rows], dtype), dev(torch.cat([torch.zeros(T, C), z], 1)[rows], dtype), dev(dbc[rows]), R, N, dev(w_dt.t()),
                         dev(b_dt), dev(a_log), dev(dsk))
    state = dev(start.clone())
    got = ops.selective_scan(*args(slice(0, T)), state, i32(starts), i32(lens), i32(slots))
    for s, (q0, n) in enumerate(zip(starts, lens)):     # each request alone, token after token
        alone = dev(start.clone())
        want = torch.cat([ops.selective_scan(*args(slice(t, t + 1)), alone, i32([0]), i32([1]), i32([slots[s]])) for t in range(q0, q0 + n)])
        close(got[q0:q0 + n], want, dtype, f"request {s} in chunks")
        close(state[slots[s]], alone[slots[s]], torch.float32, f"state of request {s}")
    assert torch.equal(state[1].cpu(), start[1]) and torch.equal(state[3].cpu(), start[3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("H,d,dv", [(2, 16, 24), (1, 40, 8), (3, 8, 70), (2, 72, 16), (2, 128, 128), (1, 136, 8)])
def test_lightning_attention_in_one_step_and_in_many(dtype, H, d, dv, chunked):
    """Token after token, and in chunks on the matrix cores (head sizes that kernel does not take run in the other)."""
    ops = ops_of(dtype)
    torch.manual_seed(d)
    n = 77
    ld = 2 * H * d + 2 * H * dv
    rows = torch.randn(n, ld).to(dtype).float()
    decay = torch.tensor([0.6, 0.95, 0.999][:H])
    q = P.silu(rows[:, :H * d].double()).view(n, H, d)
    k = P.silu(rows[:, H * d:2 * H * d].double()).view(n, H, d)
    v = P.silu(rows[:, 2 * H * d:2 * H * d + H * dv].double()).view(n, H, dv)
    S, want = torch.zeros(H, d, dv, dtype=torch.float64), torch.empty(n, H, dv, dtype=torch.float64)
    for i in range(n):
        S = decay.double()[:, None, None] * S + k[i][:, :, None] * v[i][:, None, :]
        want[i] = torch.einsum("hde,hd->he", S, q[i])
    want = want.reshape(n, H * dv)
    for cuts in ([n], [1] * n, [16, 17, 2, 32, 10]):
        state = torch.zeros(2, H, d, dv, device=DEV)
        got, at = [], 0
        for c in cuts:
            got.append(ops.lightning_attention(dev(rows[at:at + c], dtype), H, d, dv, dev(decay), state, i32([0]), i32([c]), i32([1]), chunked))
            at += c
        # in chunks the activations, the decayed scores and the state are rounded to the element type as operands
        close(torch.cat(got), want, dtype if chunked else torch.float32, f"lightning cut as {cuts[:4]}")
        close(state[1], S, dtype if chunked else torch.float32, "the state after the last token")
    w = torch.randn(H * dv)
    o = torch.cat(got)
    gated = ops.gated_rmsnorm(o, dev(rows, dtype), 2 * H * d + H * dv, dev(w), 1e-5)
    close(gated, P.rms(o.double().cpu(), 1e-5) * w.double() * torch.sigmoid(rows[:, 2 * H * d + H * dv:].double()), dtype, "gated norm")


def _attention_case(dtype, H, KV, d, dv, ps, lens_before, lens_now, window, keep, rot, talk, seed, spike=None, normed=True, tiles=False):
    """Requests with `lens_before` tokens in the cache bring `lens_now` more.  Everything goes through the two kernels,
    step by step, and is compared with the plain attention over each whole request.  `spike = (request, key position)`
    makes that key's score with every query huge (the rows are then neither normed nor rotated, which would undo it)."""
    ops = ops_of(dtype)
    g = torch.Generator().manual_seed(seed)
    S = len(lens_before)
    nq, nk, nv = H * d, KV * d, KV * dv
    tot = [a + b for a, b in zip(lens_before, lens_now)]
    qkv = [torch.randn(n, nq + nk + nv, generator=g) for n in tot]
    if spike is not None:
        s, j = spike
        u = torch.ones(d) / math.sqrt(d)
        for x in qkv:
            x[:, :nq] = u.repeat(H) + 0.1 * x[:, :nq]
        qkv[s][j, nq:nq + nk] = 30.0 * u.repeat(KV)
    qn, kn = torch.rand(nq, generator=g) + 0.5, torch.rand(nk, generator=g) + 0.5
    T_ = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g) if talk else None
    inv = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)]) if rot else None
    factor, scale = 1.3, 0.7
    pages = sum(-(-n // ps) for n in tot)
    kpool = torch.zeros(pages + 1, KV, ps, d, dtype=dtype, device=DEV)
    vpool = torch.zeros(pages + 1, KV, dv, ps, dtype=dtype, device=DEV)
    width = max(-(-n // ps) for n in tot)
    table = torch.full((S, width), -1, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()        # pages in any order
    for s in range(S):
        for p in range(-(-tot[s] // ps)):
            table[s, p] = order.pop()
    got = {}
    for phase, lens in (("before", lens_before), ("now", lens_now)):
        start = [0] * S if phase == "before" else lens_before
        live = [s for s in range(S) if lens[s] > 0]
        if not live:
            continue
        rows = torch.cat([qkv[s][start[s]:start[s] + lens[s]] for s in live])
        positions = torch.cat([torch.arange(start[s], start[s] + lens[s]) for s in live])
        slot_map = torch.cat([table[s][(torch.arange(start[s], start[s] + lens[s]) // ps)] * ps
                              + torch.arange(start[s], start[s] + lens[s]) % ps for s in live])
        q_start = [sum(lens[x] for x in live[:i]) for i in range(len(live))]
        q, _ = ops.talking_prepare(dev(rows).unsqueeze(0), dev(qn) if normed else None, dev(kn) if normed else None, 1e-5, dev(positions.int()), dev(inv) if rot else None, rot, factor,
                                   None, None, False, dev(slot_map.int()), kpool, vpool, H, KV, d, dv, ps)
        out = ops.talking_attention(q, kpool, vpool, dev(T_) if talk else None, dev(table[live]), i32(q_start), i32([start[s] for s in live]),
                                    H, KV, d, dv, ps, window, keep, scale, None if tiles == "vector" else i32([lens[s] for s in live]),
                                    tiles is True)
        if phase == "now":
            for i, s in enumerate(live):
                got[s] = out[q_start[i]:q_start[i] + lens[s]].float().cpu()
    # the plain attention over whole requests, with the same numbers
    for s in got:
        n = tot[s]
        x = qkv[s].double()
        qq = (P.rms(x[:, :nq], 1e-5) * qn.double() if normed else x[:, :nq]).view(n, H, d)
        kk = (P.rms(x[:, nq:nq + nk], 1e-5) * kn.double() if normed else x[:, nq:nq + nk]).view(n, KV, d)
        if rot:
            ang = torch.arange(n).double()[:, None] * inv.double()[None, :]
            c, sn = (torch.cos(ang) * factor)[:, None, :], (torch.sin(ang) * factor)[:, None, :]
            turn = lambda t: torch.cat([t[..., :rot // 2] * c - t[..., rot // 2:rot] * sn, t[..., rot // 2:rot] * c + t[..., :rot // 2] * sn,
                                        t[..., rot:]], -1)
            qq, kk = turn(qq), turn(kk)
        if dtype != torch.float32:      # what the kernels keep in the element type
            qq, kk = qq.to(dtype).double(), kk.to(dtype).double()
        vv = x[:, nq + nk:].view(n, KV, dv)
        vv = vv.to(dtype).double() if dtype != torch.float32 else vv
        rep = H // KV
        sc = torch.einsum("ihd,jhd->hij", qq, kk.repeat_interleave(rep, 1)) * scale
        if talk:
            sc = torch.einsum("hg,gij->hij", T_.double(), sc)
        sc = sc.masked_fill(~P.visible(n, window or n + 1, keep if window else 0)[None], float("-inf"))
        want = torch.einsum("hij,jhe->ihe", torch.softmax(sc, -1), vv.repeat_interleave(rep, 1)).reshape(n, H * dv)
        close(got[s], want[lens_before[s]:], dtype, f"attention of request {s}", scale_by=vv)
    return got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tiles", [False, True, "vector"])
@pytest.mark.parametrize("H,KV,d,dv,rot", [(4, 2, 32, 16, 16), (6, 1, 24, 40, 24), (3, 3, 8, 8, 0), (8, 8, 64, 64, 32), (5, 1, 20, 12, 4),
                                           (12, 4, 48, 80, 48), (24, 3, 16, 128, 8), (32, 32, 40, 16, 40)])
def test_talking_attention_kernels(dtype, H, KV, d, dv, rot, tiles):
    """On the matrix cores one row a block and 16 rows a block, and on the vector units (sizes that the kernel on the
    matrix cores does not take run there in every case)."""
    # prompts, portions of prompts that go on, and single decoded rows side by side; a window that crosses pages
    _attention_case(dtype, H, KV, d, dv, 16, [0, 40, 70, 5], [50, 13, 1, 1], 24, 3, rot, True, seed=H, tiles=tiles)
    _attention_case(dtype, H, KV, d, dv, 16, [0, 31], [130, 1], None, 0, rot, H % 2 == 0, seed=H + 1, tiles=tiles)    # all keys, far ones too
    _attention_case(dtype, H, KV, d, dv, 32, [3, 0, 100], [7, 9, 21], 40, 35, rot, True, seed=H + 2, tiles=tiles)   # kept tokens beyond a page
    # so many keys for so few rows that several blocks share a row's (or a tile's) keys and a second kernel merges them
    _attention_case(dtype, H, KV, d, dv, 16, [0, 200, 380], [330, 40, 1], 300, 40, rot, True, seed=H + 3, tiles=tiles)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True, "tiles", "vector"])
@pytest.mark.parametrize("edge", ["inside the window", "outside the window", "kept", "not kept", "page border", "own"])
def test_a_key_that_stands_out_shows_at_every_edge(dtype, decoded, edge):
    """One key's score is made huge: its value is the output if the row sees it, and absent if not, so a window or
    a count of kept tokens that is one off fails by the whole value."""
    window, keep, ps, n = 20, 5, 16, 64
    key = {"inside the window": n - window, "outside the window": n - window - 1, "kept": keep - 1, "not kept": keep,
           "page border": 48, "own": n - 1}[edge]
    before, now = ([n - 1], [1]) if decoded in (True, "vector") else ([0], [n])
    got = _attention_case(dtype, 4, 2, 16, 16, ps, before, now, window, keep, 0, True, seed=11, spike=(0, key), normed=False,
                          tiles=True if decoded == "tiles" else "vector" if decoded == "vector" else False)
    assert len(got) == 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_values_blend_with_the_first_layers(dtype):
    ops = ops_of(dtype)
    torch.manual_seed(1)
    T, H, KV, d, dv, ps = 6, 2, 1, 8, 8, 16
    rows = torch.randn(2, T, (H + KV) * d + KV * dv)
    kpool, vpool = (torch.zeros(2, KV, *shape, dtype=dtype, device=DEV) for shape in ((ps, d), (dv, ps)))
    slot_map, pos = i32(list(range(16, 16 + T))), i32(list(range(T)))
    _, own = ops.talking_prepare(dev(rows), None, None, 1e-5, pos, None, 0, 1.0, None, None, True, slot_map, kpool, vpool, H, KV, d, dv, ps)
    v = rows.sum(0)[:, (H + KV) * d:]
    close(own, v, torch.float32, "the layer's own values")
    close(vpool[1, 0, :, :T].T, v, dtype, "cached values, unblended")
    other = torch.randn(T, KV * dv)
    ops.talking_prepare(dev(rows), None, None, 1e-5, pos, None, 0, 1.0, dev(other), dev(torch.tensor([0.3])), False, slot_map, kpool, vpool,
                        H, KV, d, dv, ps)
    close(vpool[1, 0, :, :T].T, 0.7 * v + 0.3 * other, dtype, "cached values, blended")
    close(kpool[1, 0, :T], rows.sum(0)[:, H * d:(H + KV) * d], dtype, "keys without norm or rotation")


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
    w, cfg = U.read(model_dir)
    if dtype != torch.float32:
        w = {k: v.to(dtype).float() if v.dim() == 2 and not k.endswith((".conv", ".dt", ".A_log", ".talk")) else v for k, v in w.items()}
    return P.forward(w, cfg, tokens, torch.float64)


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
    name = "mixed"
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
def test_long_decoding_from_captured_steps(tmp_path, dtype):
    name = "narrow"
    d = U.make_dir(tmp_path, name, seed=10, sharpen=sharpen_for(dtype))
    toks = U.tokens_of(330, 50, 3)
    lm = loaded(d, dtype, max_tokens=512)
    got = U.run_schedule(lm, {"a": toks}, [[("a", 10)]] + [[("a", 1)]] * 320)["a"]
    assert U.within(got, plain_for(d, dtype, toks), dtype)
    assert len(lm.step._graphs) > 0     # the single rows ran from captured steps
    # the window groups gave pages back while it decoded, all but the first tokens' and the last ones'
    assert all(g.pool.available() >= g.pool.num_pages - 5 for g in lm.cache.groups.values())


def test_first_tokens_of_a_sequence(tmp_path):
    for name in sorted(U.CONFIGS):
        d = U.make_dir(tmp_path, name, seed=12)
        toks = U.tokens_of(4, U.CONFIGS[name]["vocab"], 1)
        lm = loaded(d, torch.float32)
        for n in (1, 2, 3, 4):
            got = U.run_schedule(lm, {"a": toks[:n]}, [[("a", n)]])["a"]
            assert U.relative_error(got, plain_for(d, torch.float32, toks[:n])) < F32, (name, n)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, dtype):
    import machserve_amd
    d = U.make_dir(tmp_path, "mixed", seed=13, sharpen=2.0)
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


def test_the_given_folder_layout_runs_through_the_trace_program(tmp_path):
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    d = U.make_dir(tmp_path, "mixed", seed=14, sharpen=2.0)
    toks = U.tokens_of(50, 97, 2)
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
    got = torch.from_numpy(np.concatenate([np.fromfile(out / "0.f32", dtype="<f4"), np.fromfile(out / "1.f32", dtype="<f4")]).reshape(3, 97))
    assert U.relative_error(got, want[[0, 32, 49]]) < F32


def test_command_line_generates_from_a_folder_and_from_a_configuration(tmp_path):
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    d = U.make_dir(tmp_path, "stateful", seed=15)
    w, cfg = U.read(d)
    prompt = U.tokens_of(9, 61, 4)
    cmd = [sys.executable, os.path.join(root, "bin", "machserve"), "--max-new", "5", "--dtype", "f32", "--tpp", "16", "--prompt-ids"]
    r = subprocess.run(cmd + [",".join(map(str, prompt)), "--model", d], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.split()] == P.greedy_generate(w, cfg, prompt, 5, torch.float64)
    path = tmp_path / "config.json"
    path.write_text(json.dumps(U.CONFIGS["narrow"]))
    r = subprocess.run(cmd + ["7,49,0,12", "--random-config", str(path), "--weights-seed", "3"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert len(r.stdout.split()) == 5 and all(0 <= int(t) < 50 for t in r.stdout.split())
