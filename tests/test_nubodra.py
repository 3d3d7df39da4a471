"""Nubodra without a GPU: the configuration, the plain model's own mechanisms against closed forms, and the engine's host
side (parts, cache manager with pages and state slots together, step function, scheduler) over CPU stand-ins for the
kernels, against the plain model."""
import json
import math

import pytest
import torch

import nubodra_util as U
from emulated_ops import EmulatedOps
from plain import nubodra_plain as P

from machserve_amd.config import ConfigError, NubodraConfig, config_from_dict
from machserve_amd.engine.loading import load_model

# The stand-ins leave a product of few rows as two partial sums, one of them noise of order one: 32-bit rounding of that
# noise, through sharpened softmaxes, is what this bound allows.  A key that is missing or one too many, a lost state or
# a sink left out is off by a hundred times more.
TOL = 5e-4


def loaded(model_dir, page_size=16, max_tokens=512, max_requests=4, num_pages=None):
    return load_model(model_dir, dtype="float32", device="cpu", ops=EmulatedOps(torch.float32), page_size=page_size,
                      max_tokens=max_tokens, max_requests=max_requests, use_graphs=False, num_pages=num_pages)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_configuration_round_trip_and_plan(name):
    cfg = config_from_dict(U.CONFIGS[name])
    assert isinstance(cfg, NubodraConfig)
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    spec = cfg.to_spec()
    assert len(spec.layers) == len(U.CONFIGS[name]["layers"]) and all(l.block == "parallel" for l in spec.layers)
    names = [n for n, _, _ in cfg.random_tensor_plan()]
    assert len(set(names)) == len(names) and names[0] == "embed" and names[-1] == "head"
    # a layer that reads another's cache has no down projection of keys
    for i, layer in enumerate(U.CONFIGS[name]["layers"]):
        assert (f"l{i}.mix.dkv" in names) == (layer["type"] == "latent_attention" and "kv_from" not in layer["mixer"])


def test_configuration_errors_name_the_key():
    def broken(change):
        raw = json.loads(json.dumps(U.CONFIGS["pair"]))
        change(raw)
        return raw
    with pytest.raises(ConfigError, match=r"layers\[0\]\.mixer\.kv_rank"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"].pop("kv_rank")))
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=6)))
    with pytest.raises(ConfigError, match="rwkv"):
        config_from_dict(broken(lambda r: r["layers"][1].update(type="rwkv")))
    with pytest.raises(ConfigError, match="kv_from"):      # a layer cannot read a later layer, itself or one that reads
        config_from_dict(broken(lambda r: r["layers"][2]["mixer"].update(kv_from=2)))
    with pytest.raises(ConfigError, match="kv_from"):      # nor an attention of the other kind
        config_from_dict(broken(lambda r: r["layers"][2]["mixer"].update(kv_from=1)))
    with pytest.raises(ConfigError, match="kv_rank"):      # and the two latents must be alike
        config_from_dict(broken(lambda r: r["layers"][2]["mixer"].update(kv_rank=32)))
    with pytest.raises(ConfigError, match="kv_heads"):
        config_from_dict(broken(lambda r: r["layers"][1]["mixer"].update(kv_heads=3)))
    with pytest.raises(ConfigError, match="vdim"):         # the values are the keys
        config_from_dict(broken(lambda r: r["layers"][1]["mixer"].update(vdim=8)))
    with pytest.raises(ConfigError, match="norm"):
        config_from_dict(broken(lambda r: r.pop("norm")))


# ------------------------------------------------------------------ the plain mechanisms against closed forms
def test_layer_norm_and_unit_norm():
    x = torch.randn(5, 12, dtype=torch.float64) * 3 + 1
    w, b = torch.randn(12, dtype=torch.float64), torch.randn(12, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (12,), w, b, 1e-5))
    y = P.rms(x, 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64))


def test_convolution_is_causal_and_starts_from_zeros():
    u = torch.randn(9, 3, dtype=torch.float64)
    w = torch.randn(3, 4, dtype=torch.float64)
    y = P.causal_conv(u, w)
    assert torch.allclose(y[0], w[:, 3] * u[0])                       # before the start: zeros
    assert torch.allclose(y[5], sum(w[:, j] * u[5 - 3 + j] for j in range(4)))
    u2 = u.clone()
    u2[6:] += 1.0
    assert torch.allclose(P.causal_conv(u2, w)[:6], y[:6])            # nothing of the future
    assert torch.allclose(P.causal_conv(u, w[:, 3:]), u * w[:, 3])    # one tap: a scaling


def test_query_temperature_steps_with_the_position():
    t = P.query_temperature(13, 0.5, 4, torch.float64)
    assert t[0] == 1.0 and t[2] == 1.0                                # floor((p + 1) / 4) = 0 up to p = 2
    assert math.isclose(float(t[3]), 1 + 0.5 * math.log(2.0)) and math.isclose(float(t[6]), 1 + 0.5 * math.log(2.0))
    assert math.isclose(float(t[11]), 1 + 0.5 * math.log(4.0))
    assert math.isclose(float(P.query_temperature(3, 2.0, 1, torch.float64)[2]), 1 + 2.0 * math.log(4.0))


def test_sink_only_takes_weight():
    s = torch.randn(2, 4, 4, dtype=torch.float64)
    p = P.causal_softmax(s)
    assert torch.allclose(p.sum(-1), torch.ones(2, 4, dtype=torch.float64)) and float(p[0, 1, 2]) == 0.0
    sink = torch.tensor([0.3, -50.0], dtype=torch.float64)
    ps = P.causal_softmax(s, sink)
    assert torch.allclose(ps[1], p[1])                                # a sink far below every score changes nothing
    first = 1.0 / (1.0 + math.exp(0.3 - float(s[0, 0, 0])))            # one key and the sink
    assert math.isclose(float(ps[0, 0, 0]), first)
    assert torch.allclose(ps[0] / ps[0].sum(-1, keepdim=True), p[0])  # the keys share what the sink leaves as before


def test_rotation_of_neighbours_and_scaled_frequencies():
    rot = {"base": 100.0, "dims": 4}
    x = torch.tensor([[1.0, 0.0, 0.0, 2.0, 7.0]], dtype=torch.float64).repeat(3, 1)
    y = P.rotate_interleaved(x, torch.arange(3), rot)
    assert torch.allclose(y[0], x[0]) and torch.allclose(y[:, 4], x[:, 4])
    assert torch.allclose(y[2, :2], torch.tensor([math.cos(2.0), math.sin(2.0)], dtype=torch.float64))
    assert torch.allclose(y[2, 2:4], torch.tensor([-2 * math.sin(0.2), 2 * math.cos(0.2)], dtype=torch.float64))
    f, factor = P.rotary_frequencies({"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}})
    plain, one = P.rotary_frequencies({"base": 10000.0, "dims": 8})
    assert one == 1.0 and math.isclose(factor, 0.1 * math.log(4.0) + 1.0)
    assert math.isclose(float(f[0]), float(plain[0])) and math.isclose(float(f[3]), float(plain[3]) / 4.0)  # fast pairs stay, slow ones slow down
    # a relative position is all a score depends on
    q, k = torch.randn(1, 4, dtype=torch.float64), torch.randn(1, 4, dtype=torch.float64)
    a = (P.rotate_interleaved(q, torch.tensor([9]), rot) * P.rotate_interleaved(k, torch.tensor([4]), rot)).sum()
    b = (P.rotate_interleaved(q, torch.tensor([25]), rot) * P.rotate_interleaved(k, torch.tensor([20]), rot)).sum()
    assert math.isclose(float(a), float(b), rel_tol=1e-9)


def test_plain_model_whole_equals_its_prefixes(tmp_path):
    d = U.make_dir(tmp_path, "pair", seed=1)
    w, cfg = U.read(d)
    toks = U.tokens_of(20, 97, 0)
    whole = P.forward(w, cfg, toks)
    for n in (1, 2, 7, 19):
        assert torch.allclose(P.forward(w, cfg, toks[:n])[-1], whole[n - 1], atol=1e-9)


# ------------------------------------------------------------------ the engine's host side over CPU stand-ins
def _cut(rid, n, sizes):
    out, at, k = [], 0, 0
    while at < n:
        c = min(sizes[k % len(sizes)], n - at)
        out.append([(rid, c)])
        at, k = at + c, k + 1
    return out


@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_any_cut_of_a_prompt_equals_the_plain_model(tmp_path, name):
    d = U.make_dir(tmp_path, name, seed=3)
    n = 70
    toks = U.tokens_of(n, U.CONFIGS[name]["vocab"], 5)
    want = U.plain_logits(d, toks)
    lm = loaded(d)
    for what, schedule in {"whole": [[("a", n)]], "token by token": [[("a", 1)]] * n,
                           "portions down to two tokens": _cut("a", n, [2, 17, 3, 2, 16, 1, 1, 15, 2])}.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.relative_error(got, want) < TOL, what
    lm.cache.check()


def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(tmp_path):
    d = U.make_dir(tmp_path, "pair", seed=4)
    reqs = {"a": U.tokens_of(50, 97, 1), "b": U.tokens_of(1, 97, 2), "c": U.tokens_of(33, 97, 3), "d": U.tokens_of(40, 97, 4)}
    schedule = [[("b", 1), ("a", 17), ("c", 3)], [("a", 1), ("c", 30)], [("a", 2), ("d", 15)], [("a", 1), ("d", 1)], [("a", 29), ("d", 24)]]
    lm = loaded(d, max_requests=3, num_pages=8)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.relative_error(got[i], U.plain_logits(d, toks)) < TOL, i
    lm.cache.check()
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


def test_a_slot_used_again_starts_its_convolution_from_zeros(tmp_path):
    d = U.make_dir(tmp_path, "odd", seed=5)
    lm = loaded(d, max_requests=1)
    a, b = U.tokens_of(9, 61, 1), U.tokens_of(6, 61, 2)
    U.run_schedule(lm, {"a": a}, [[("a", 9)]])
    got = U.run_schedule(lm, {"b": b}, [[("b", 2)], [("b", 4)]])["b"]
    assert U.relative_error(got, U.plain_logits(d, b)) < TOL


def test_groups_of_the_cache(tmp_path):
    lm = loaded(U.make_dir(tmp_path, "odd", seed=6))
    # the attention layers' pages, and a group for each width of latent; the layer that reads another's cache has none
    assert len(lm.cache.groups) == 3
    assert sum(len(g.spec.layers) for g in lm.cache.groups.values()) == 4
    assert all(g.spec.kv_heads == 1 for name, g in lm.cache.groups.items() if "kv1x" in name)


def test_greedy_generation_through_the_scheduler(tmp_path):
    from machserve_amd.engine import Engine
    d = U.make_dir(tmp_path, "pair", seed=7)
    w, cfg = U.read(d)
    prompts = [U.tokens_of(n, 97, n) for n in (5, 19, 1, 30)]
    lm = loaded(d, max_requests=3, max_tokens=256)
    engine = Engine(lm, max_batch_tokens=24, chunk_size=8, max_running=3, freeze_gc=False)
    got = engine.generate(prompts, max_new=5)
    for p, g in zip(prompts, got):
        assert g == P.greedy_generate(w, cfg, p, 5, torch.float64)
    lm.cache.check()
