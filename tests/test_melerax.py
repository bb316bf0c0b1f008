"""Melerax without a GPU: the configuration, the plain model's own mechanisms against closed forms, and the engine's host
side (parts, cache manager with pages and state slots together, step function, scheduler) over CPU stand-ins for the
kernels, against the plain model."""
import json
import math

import pytest
import torch

import melerax_util as U
from emulated_ops import EmulatedOps
from plain import melerax_plain as P

from machserve_amd.config import ConfigError, MeleraxConfig, config_from_dict
from machserve_amd.engine.loading import load_model

# The stand-ins leave a product of few rows as two partial sums, one of them noise of order one: 32-bit rounding of that
# noise, through sharpened softmaxes, is what this bound allows.  A key that is missing or one too many, a lost state or
# a wrong chunk is off by a hundred times more.
TOL = 5e-4
F64 = torch.float64


def loaded(model_dir, page_size=16, max_tokens=512, max_requests=4, num_pages=None):
    return load_model(model_dir, dtype="float32", device="cpu", ops=EmulatedOps(torch.float32), page_size=page_size,
                      max_tokens=max_tokens, max_requests=max_requests, use_graphs=False, num_pages=num_pages)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_configuration_round_trip_and_plan(name):
    cfg = config_from_dict(U.CONFIGS[name])
    assert isinstance(cfg, MeleraxConfig)
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    spec = cfg.to_spec()
    assert len(spec.layers) == len(U.CONFIGS[name]["layers"]) and all(l.block == "postnorm" for l in spec.layers)
    names = [n for n, _, _ in cfg.random_tensor_plan()]
    assert len(set(names)) == len(names) and names[0] == "embed" and names[-1] == "head"
    for i, layer in enumerate(U.CONFIGS[name]["layers"]):
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
        assert (f"l{i}.mix.left.q.conv" in names) == (layer["type"] == "parallel")
        assert (f"l{i}.mlp.router" in names) == (layer["mlp"] is not None and layer["mlp"]["kind"] == "moe")


def test_configuration_errors_name_the_key():
    def broken(change):
        raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
        change(raw)
        return raw
    with pytest.raises(ConfigError, match=r"layers\[0\]\.mixer\.left\.kv_heads"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"]["left"].pop("kv_heads")))
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=7)))
    with pytest.raises(ConfigError, match="mamba"):
        config_from_dict(broken(lambda r: r["layers"][1].update(type="mamba")))
    with pytest.raises(ConfigError, match="blocks"):
        config_from_dict(broken(lambda r: r["layers"][2]["mixer"].update(blocks=3)))
    with pytest.raises(ConfigError, match="top"):
        config_from_dict(broken(lambda r: r["layers"][1]["mlp"]["router"].update(top=9)))
    with pytest.raises(ConfigError, match="kind"):
        config_from_dict(broken(lambda r: r["layers"][0]["mlp"].update(kind="glu")))
    with pytest.raises(ConfigError, match="norm"):
        config_from_dict(broken(lambda r: r.pop("norm")))
    with pytest.raises(ConfigError, match="buckets"):
        config_from_dict(broken(lambda r: r["embedding"]["bigram"].pop("buckets")))


# ------------------------------------------------------------------ the plain mechanisms against closed forms
def test_pair_rows_and_the_first_token():
    rows = P.bigram_rows([5, 9, 9, 0], 7, 3, 53)
    assert list(map(int, rows)) == [53, (5 * 7 + 9 * 3) % 53, (9 * 7 + 9 * 3) % 53, (9 * 7) % 53]


def test_convolution_is_causal_and_starts_from_zeros():
    u, w = torch.randn(9, 3, dtype=F64), torch.randn(3, 4, dtype=F64)
    y = P.causal_conv(u, w)
    assert torch.allclose(y[0], w[:, 3] * u[0])
    assert torch.allclose(y[5], sum(w[:, j] * u[5 - 3 + j] for j in range(4)))
    u2 = u.clone()
    u2[6:] += 1.0
    assert torch.allclose(P.causal_conv(u2, w)[:6], y[:6])


def test_rotation_of_neighbours_leaves_the_rest_and_keeps_lengths():
    x = torch.randn(6, 2, 10, dtype=F64)
    y = P.rotate_neighbours(x, {"base": 100.0, "dims": 6})
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., :6].pow(2).sum(-1), x[..., :6].pow(2).sum(-1))
    p, i = 4, 1
    a = p * 100.0 ** (-2 * i / 6)
    assert torch.allclose(y[p, 0, 2], x[p, 0, 2] * math.cos(a) - x[p, 0, 3] * math.sin(a))
    assert torch.allclose(y[p, 0, 3], x[p, 0, 3] * math.cos(a) + x[p, 0, 2] * math.sin(a))


def test_chunks_are_counted_from_position_zero():
    see = P.chunk_visible(10, 4)
    assert see[3].tolist() == [True] * 4 + [False] * 6
    assert see[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert see[9].tolist() == [False] * 8 + [True, True]


def test_recurrence_in_closed_form_for_constant_gates():
    # with zero gate maps r = i = 1/2 whatever u is: S_n = sum_j a^(n-j) sqrt(1 - a^2) u_j / 2
    n, c = 7, 4
    t = {"y": torch.zeros(c, 3, dtype=F64), "y.b": torch.full((c,), 0.8, dtype=F64), "x": torch.randn(c, 3, dtype=F64), "x.b": torch.zeros(c, dtype=F64),
         "conv": torch.tensor([[0.0, 1.0]] * c, dtype=F64), "conv.b": torch.zeros(c, dtype=F64), "ra": torch.zeros(2, 2, 2, dtype=F64),
         "ra.b": torch.zeros(2, 2, dtype=F64), "ri": torch.zeros(2, 2, 2, dtype=F64), "ri.b": torch.zeros(2, 2, dtype=F64),
         "lam": torch.randn(c, dtype=F64), "o": torch.eye(c, dtype=F64)}
    h = torch.randn(n, 3, dtype=F64)
    got = P.rglru(h, t, {"width": c, "blocks": 2, "conv": 2})
    a = torch.exp(-8.0 * 0.5 * torch.nn.functional.softplus(t["lam"]))
    u = h @ t["x"].T
    want = torch.stack([sum(a ** (i - j) * torch.sqrt(1 - a * a) * 0.5 * u[j] for j in range(i + 1)) for i in range(n)]) * P.gelu_tanh(torch.tensor(0.8, dtype=F64))
    assert torch.allclose(got, want)


def test_routing_takes_the_largest_logits_and_weighs_them_among_themselves():
    t = {"router": torch.eye(4, dtype=F64), "router.b": torch.tensor([0.0, 0.0, 0.0, 5.0], dtype=F64)}
    h = torch.tensor([[3.0, 1.0, 2.0, -9.0], [0.0, 0.0, 0.0, 0.0]], dtype=F64)
    idx, w = P.route(h, t, 2)
    assert idx[0].tolist() == [0, 2] and idx[1][0] == 3
    assert torch.allclose(w[0], torch.softmax(torch.tensor([3.0, 2.0], dtype=F64), 0))


def test_plain_model_whole_equals_its_prefixes(tmp_path):
    d = U.make_dir(tmp_path, "mixed", seed=1)
    w, cfg = U.read(d)
    toks = U.tokens_of(40, 97, 0)
    whole = P.forward(w, cfg, toks)
    for n in (1, 2, 7, 17, 39):
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
    d = U.make_dir(tmp_path, "mixed", seed=4)
    reqs = {"a": U.tokens_of(50, 97, 1), "b": U.tokens_of(1, 97, 2), "c": U.tokens_of(33, 97, 3), "d": U.tokens_of(40, 97, 4)}
    schedule = [[("b", 1), ("a", 17), ("c", 3)], [("a", 1), ("c", 30)], [("a", 2), ("d", 15)], [("a", 1), ("d", 1)], [("a", 29), ("d", 24)]]
    lm = loaded(d, max_requests=3, num_pages=8)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.relative_error(got[i], U.plain_logits(d, toks)) < TOL, i
    lm.cache.check()
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


def test_a_slot_used_again_starts_every_state_from_zeros(tmp_path):
    """The previous token, both convolutions, both recurrences and the token before: all of them belong to the slot."""
    d = U.make_dir(tmp_path, "odd", seed=5)
    lm = loaded(d, max_requests=1)
    a, b = U.tokens_of(9, 61, 1), U.tokens_of(6, 61, 2)
    U.run_schedule(lm, {"a": a}, [[("a", 9)]])
    got = U.run_schedule(lm, {"b": b}, [[("b", 2)], [("b", 4)]])["b"]
    assert U.relative_error(got, U.plain_logits(d, b)) < TOL


def test_what_the_layers_ask_of_the_cache(tmp_path):
    lm = loaded(U.make_dir(tmp_path, "mixed", seed=6))
    # two attention layers with heads of different sizes: two groups of all keys; every layer and the embedding keep a state
    assert len(lm.cache.groups) == 2 and all(g.spec.window is None for g in lm.cache.groups.values())
    states = lm.cache.states
    assert (5, 0) in states and states[(5, 0)].dtype == torch.int32                     # the embedding's previous token
    assert set(states[(1, 0)].shapes) == {"prev", "wkv"} and set(states[(2, 0)].shapes) == {"lru", "conv"}
    assert states[(0, 1)].shapes == {"conv": (2, 4 * 16 + 2 * 16 + 2 * 24)}            # the attention's q, k and v before the taps
    assert set(states[(0, 2)].shapes) == {"lru", "conv"}


def test_greedy_generation_through_the_scheduler(tmp_path):
    from machserve_amd.engine import Engine
    d = U.make_dir(tmp_path, "mixed", seed=7)
    w, cfg = U.read(d)
    prompts = [U.tokens_of(n, 97, n) for n in (5, 19, 1, 30)]
    lm = loaded(d, max_requests=3, max_tokens=256)
    engine = Engine(lm, max_batch_tokens=24, chunk_size=8, max_running=3, freeze_gc=False)
    got = engine.generate(prompts, max_new=5)
    for p, g in zip(prompts, got):
        assert g == P.greedy_generate(w, cfg, p, 5, torch.float64)
    lm.cache.check()
