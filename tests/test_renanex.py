"""Renanex without a GPU: the configuration, the plain model's own mechanisms, and the engine's host side (parts, cache
manager with state slots and kept first pages, step function, scheduler) over CPU stand-ins for the kernels, against the
plain model."""
import json
import math

import pytest
import torch

import renanex_util as U
from emulated_ops import EmulatedOps
from plain import renanex_plain as P

from machserve_amd.config import ConfigError, RenanexConfig, config_from_dict
from machserve_amd.engine.loading import load_model


# The stand-ins leave a product of few rows as two partial sums, one of them noise of order one, as the kernels may
# leave sums of any split: 32-bit rounding of that noise, through sharpened softmaxes, is what this bound allows.  A key
# that is missing or one too many, or a state that is lost, is off by a hundred times more.
TOL = 5e-4


def loaded(model_dir, page_size=16, max_tokens=512, max_requests=4, num_pages=None):
    return load_model(model_dir, dtype="float32", device="cpu", ops=EmulatedOps(torch.float32), page_size=page_size,
                      max_tokens=max_tokens, max_requests=max_requests, use_graphs=False, num_pages=num_pages)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_configuration_round_trip_and_plan(name):
    cfg = config_from_dict(U.CONFIGS[name])
    assert isinstance(cfg, RenanexConfig)
    again = config_from_dict(json.loads(json.dumps(cfg.to_dict())))
    assert again == cfg
    spec = cfg.to_spec()
    assert len(spec.layers) == len(U.CONFIGS[name]["layers"])
    names = [n for n, _, _ in cfg.random_tensor_plan()]
    assert len(set(names)) == len(names) and names[0] == "embed" and names[-1] == "head"


def test_configuration_errors_name_the_key():
    raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
    del raw["layers"][1]["mixer"]["dt_rank"]
    with pytest.raises(ConfigError, match=r"layers\[1\]\.mixer\.dt_rank"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
    raw["layers"][0]["mixer"]["rot"]["dims"] = 34
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
    raw["layers"][2]["type"] = "rwkv"
    with pytest.raises(ConfigError, match="rwkv"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
    raw["layers"][3]["mixer"]["vdim"] = 8      # blending layers must agree on the values' shape
    with pytest.raises(ConfigError, match="v_mix"):
        config_from_dict(raw)


def test_blend_roles_follow_the_order_of_layers():
    spec = config_from_dict(U.CONFIGS["mixed"]).to_spec()
    assert [getattr(layer.mixer, "value_blend", "-") for layer in spec.layers] == ["source", "-", "-", "blend", None]
    assert spec.layers[3].feed_forward is None and spec.layers[3].feed_forward_norm is None


# ------------------------------------------------------------------ the plain model's mechanisms, each alone
def test_plain_visibility():
    m = P.visible(12, 4, 2)
    assert m[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert m[3].tolist() == [True] * 4 + [False] * 8
    assert m[5].tolist() == [True, True, True, True, True, True] + [False] * 6   # 2 kept, then 2..5
    assert P.visible(6, 100, 0).tolist() == torch.tril(torch.ones(6, 6)).bool().tolist()


def test_plain_rotation_of_a_part_of_the_head():
    rot = {"base": 100.0, "dims": 4}
    x = torch.randn(5, 2, 6, dtype=torch.float64)
    y = P.rotate(x, torch.arange(5), rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., :4].norm(dim=-1), x[..., :4].norm(dim=-1))
    a = 3 * 100.0 ** (-2 / 4)     # pair (1, 3) at position 3
    assert torch.allclose(y[3, 0, 1], x[3, 0, 1] * math.cos(a) - x[3, 0, 3] * math.sin(a))
    assert torch.allclose(y[3, 0, 3], x[3, 0, 3] * math.cos(a) + x[3, 0, 1] * math.sin(a))
    # scores depend on the distance only
    q, k = torch.randn(1, 1, 6, dtype=torch.float64), torch.randn(1, 1, 6, dtype=torch.float64)
    s = lambda i, j: (P.rotate(q, torch.tensor([i]), rot) * P.rotate(k, torch.tensor([j]), rot)).sum()
    assert torch.allclose(s(9, 4), s(25, 20))


def test_plain_scaled_frequencies():
    rot = {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    f, factor = P.rotary_frequencies(rot)
    plain, _ = P.rotary_frequencies({"base": 10000.0, "dims": 16})
    index = lambda turns: 16 * math.log(64 / (2 * math.pi * turns)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(index(8.0)), 0), min(math.ceil(index(1.0)), 15)
    assert factor == pytest.approx(0.1 * math.log(4.0) + 1.0)
    for i in range(8):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        assert float(f[i]) == pytest.approx(float(plain[i]) * (ramp / 4.0 + 1.0 - ramp))
    assert float(f[0]) == pytest.approx(1.0) and float(f[7]) == pytest.approx(float(plain[7]) / 4.0)


def test_plain_recurrences_equal_their_closed_forms():
    torch.manual_seed(0)
    n, H, d, dv = 7, 2, 3, 4
    m = {"heads": H, "dim": d, "vdim": dv, "decay": [0.5, 0.9]}
    t = {k: torch.randn(s, 5, dtype=torch.float64) for k, s in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv))}
    t["o"], t["norm"] = torch.eye(H * dv, dtype=torch.float64), torch.ones(H * dv, dtype=torch.float64)
    h = torch.randn(n, 5, dtype=torch.float64)
    got = P.lightning(h, t, m, 1e-6)
    q, k, v = (P.silu(h @ t[x].T).view(n, H, -1) for x in "qkv")
    o = torch.zeros(n, H, dv, dtype=torch.float64)
    for i in range(n):
        for j in range(i + 1):
            for hh in range(H):
                o[i, hh] += m["decay"][hh] ** (i - j) * (q[i, hh] @ k[j, hh]) * v[j, hh]
    want = P.rms(o.reshape(n, -1), 1e-6) * torch.sigmoid(h @ t["g"].T)
    assert torch.allclose(got, want)
    # the scan: a constant input and step size give a geometric series
    C, N, R = 2, 3, 1
    mm = {"inner": C, "state": N, "dt_rank": R, "conv": 1}
    tt = {"in": torch.zeros(2 * C, 5, dtype=torch.float64), "conv": torch.ones(C, 1, dtype=torch.float64),
          "conv.b": torch.full((C,), 2.0, dtype=torch.float64), "x": torch.zeros(R + 2 * N, C, dtype=torch.float64),
          "dt": torch.zeros(C, R, dtype=torch.float64), "dt.b": torch.zeros(C, dtype=torch.float64),
          "A_log": torch.zeros(C, N, dtype=torch.float64), "D": torch.ones(C, dtype=torch.float64), "o": torch.eye(C, dtype=torch.float64)}
    y = P.mamba1(torch.zeros(4, 5, dtype=torch.float64), tt, mm)
    assert torch.allclose(y, torch.zeros(4, C, dtype=torch.float64))   # z = 0 gates everything away
    tt["in"][C:] = 1.0
    hh = torch.ones(4, 5, dtype=torch.float64)
    x = P.silu(torch.tensor(2.0, dtype=torch.float64))                  # B = C = 0: only the skip path D x is left
    assert torch.allclose(P.mamba1(hh, tt, mm), (x * P.silu(torch.tensor(5.0, dtype=torch.float64))).expand(4, C))


# ------------------------------------------------------------------ the engine's host side against the plain model
SCHEDULES = {
    "whole": lambda n: [[("a", n)]],
    "token by token": lambda n: [[("a", 1)] for _ in range(n)],
    "portions": lambda n: _cut("a", n, [2, 17, 3, 16, 5, 2, 31, 1, 1, 2]),
}


def _cut(rid, n, sizes):
    out, at, k = [], 0, 0
    while at < n:
        c = min(sizes[k % len(sizes)], n - at)
        out.append([(rid, c)])
        at, k = at + c, k + 1
    return out


@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_any_cut_of_a_prompt_equals_the_plain_model(tmp_path, name, schedule):
    d = U.make_dir(tmp_path, name, seed=3, sharpen=2.0)
    toks = U.tokens_of(70, U.CONFIGS[name]["vocab"], 5)
    want = U.plain_logits(d, toks)
    got = U.run_schedule(loaded(d), {"a": toks}, SCHEDULES[schedule](len(toks)))["a"]
    assert U.relative_error(got, want) < TOL


def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(tmp_path):
    name = "mixed"
    d = U.make_dir(tmp_path, name, seed=4, sharpen=2.0)
    vocab = U.CONFIGS[name]["vocab"]
    reqs = {"a": U.tokens_of(60, vocab, 1), "b": U.tokens_of(1, vocab, 2), "c": U.tokens_of(37, vocab, 3),
            "d": U.tokens_of(50, vocab, 4), "e": U.tokens_of(33, vocab, 5)}
    schedule = [[("b", 1), ("a", 20), ("c", 5)], [("a", 1), ("c", 30)], [("a", 2), ("c", 2), ("d", 17)],
                [("d", 1), ("e", 16)], [("a", 30), ("e", 1), ("d", 2)], [("a", 7), ("d", 30), ("e", 16)]]
    # two slots more than one request needs at a time, pages for the live requests only: both are handed out again
    lm = loaded(d, page_size=16, max_requests=3, num_pages=12)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.relative_error(got[i], U.plain_logits(d, toks)) < TOL, i
    lm.cache.check()
    assert lm.cache.live_requests() == []
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


def test_a_window_group_gives_pages_back_but_never_those_of_the_first_tokens(tmp_path):
    d = U.make_dir(tmp_path, "narrow", seed=1)
    lm = loaded(d, page_size=16, max_tokens=400)
    assert sorted(lm.cache.groups) == ["window19+first1", "window8+first20"]
    toks = U.tokens_of(150, 50, 9)
    from machserve_amd.engine.step import StepEntry
    slot = lm.cache.admit()
    for at in range(0, 150, 30):
        lm.step([StepEntry(slot, toks[at:at + 30], [])])
    first20 = lm.cache.table("window8+first20", slot)
    first1 = lm.cache.table("window19+first1", slot)
    # 150 tokens written; the next row is at 150: a window of 8 reaches back to 143 (page 8), one of 19 to 132 (page 8)
    assert [p >= 0 for p in first20] == [True, True] + [False] * 6 + [True, True]
    assert [p >= 0 for p in first1] == [True] + [False] * 7 + [True, True]
    lm.cache.check()
    lm.cache.release(slot)


def test_a_model_of_states_only_takes_no_pages(tmp_path):
    d = U.make_dir(tmp_path, "stateful", seed=2)
    lm = loaded(d)
    assert lm.cache.groups == {}
    toks = U.tokens_of(40, 61, 2)
    got = U.run_schedule(lm, {"a": toks, "b": toks[:9]}, [[("a", 13), ("b", 2)], [("a", 1), ("b", 7)], [("a", 26)]])
    want = U.plain_logits(d, toks)
    assert U.relative_error(got["a"], want) < TOL and U.relative_error(got["b"], want[:9]) < TOL


def test_a_slot_that_is_used_again_starts_from_zero_state(tmp_path):
    d = U.make_dir(tmp_path, "stateful", seed=5)
    lm = loaded(d, max_requests=1)
    a, b = U.tokens_of(25, 61, 1), U.tokens_of(12, 61, 2)
    got_a = U.run_schedule(lm, {"a": a}, [[("a", 25)]])["a"]
    got_b = U.run_schedule(lm, {"b": b}, [[("b", 5)], [("b", 7)]])["b"]   # the same slot, after a
    assert U.relative_error(got_a, U.plain_logits(d, a)) < TOL
    assert U.relative_error(got_b, U.plain_logits(d, b)) < TOL


def test_greedy_generation_through_the_scheduler(tmp_path):
    from machserve_amd.engine import Engine
    d = U.make_dir(tmp_path, "mixed", seed=6, sharpen=2.0)
    w, cfg = U.read(d)
    prompts = [U.tokens_of(n, 97, n) for n in (3, 21, 1, 40)]
    lm = loaded(d, max_requests=3, max_tokens=256)
    engine = Engine(lm, max_batch_tokens=24, chunk_size=16, max_running=3, freeze_gc=False)
    got = engine.generate(prompts, max_new=6)
    for p, g in zip(prompts, got):
        assert g == P.greedy_generate(w, cfg, p, 6, torch.float64)
    lm.cache.check()
