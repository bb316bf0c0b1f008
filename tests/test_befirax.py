"""Befirax without a GPU: the configuration, the plain model's own mechanisms against closed forms, and the engine's host
side (parts, cache manager with pages, windows and state slots together, step function, scheduler) over CPU stand-ins
for the kernels, against the plain model."""
import json
import math

import pytest
import torch

import befirax_util as U
from emulated_ops import EmulatedOps
from plain import befirax_plain as P

from machserve_amd.config import BefiraxConfig, ConfigError, config_from_dict
from machserve_amd.engine.loading import load_model

# The stand-ins leave a product of few rows as two partial sums, one of them noise of order one: 32-bit rounding of that
# noise, through sharpened softmaxes, is what this bound allows.  A key that is missing or one too many, a lost state or
# a window that is off by one is off by a hundred times more.
TOL = 5e-4
F64 = torch.float64


def loaded(model_dir, page_size=16, max_tokens=512, max_requests=4, num_pages=None):
    return load_model(model_dir, dtype="float32", device="cpu", ops=EmulatedOps(torch.float32), page_size=page_size,
                      max_tokens=max_tokens, max_requests=max_requests, use_graphs=False, num_pages=num_pages)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(U.CONFIGS))
def test_configuration_round_trip_and_plan(name):
    raw = U.CONFIGS[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, BefiraxConfig)
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    spec = cfg.to_spec()
    block = "multistream" if "streams" in raw else "prenorm"
    assert len(spec.layers) == len(raw["layers"]) and all(l.block == block for l in spec.layers) and spec.streams == raw.get("streams")
    names = [n for n, _, _ in cfg.random_tensor_plan()]
    assert len(set(names)) == len(names) and names[0] == "embed" and names[-1] == "final.norm"
    for i, layer in enumerate(raw["layers"]):
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None) == (f"l{i}.mlp.router" in names)
        assert (f"l{i}.hc1.mix" in names) == ("streams" in raw) and (f"l{i}.hc2.mix" in names) == ("streams" in raw and layer["mlp"] is not None)
        assert (f"l{i}.mix.k" in names) == (layer["type"] == "attention" and "kv_from" not in layer["mixer"])
        assert (f"l{i}.mix.q.conv" in names) == (layer["type"] == "attention" and layer["mixer"].get("conv", 0) > 0)
        assert (f"l{i}.mix.dt_bias" in names) == (layer["type"] == "mamba2")


def test_configuration_errors_name_the_key():
    def broken(change):
        raw = json.loads(json.dumps(U.CONFIGS["mixed"]))
        change(raw)
        return raw
    with pytest.raises(ConfigError, match=r"layers\[0\]\.mixer\.kv_heads"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"].pop("kv_heads")))
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7)))
    with pytest.raises(ConfigError, match="rot_dim"):
        config_from_dict(broken(lambda r: r["layers"][2]["mixer"]["rot"].update(dims=4)))
    with pytest.raises(ConfigError, match="mamba"):
        config_from_dict(broken(lambda r: r["layers"][1].update(type="mamba")))
    with pytest.raises(ConfigError, match="groups"):
        config_from_dict(broken(lambda r: r["layers"][1]["mixer"].update(groups=3)))
    with pytest.raises(ConfigError, match="norm_groups"):
        config_from_dict(broken(lambda r: r["layers"][1]["mixer"].update(norm_groups=5)))
    with pytest.raises(ConfigError, match="top"):
        config_from_dict(broken(lambda r: r["layers"][1]["mlp"]["router"].update(top=9)))
    with pytest.raises(ConfigError, match="kind"):
        config_from_dict(broken(lambda r: r["layers"][0]["mlp"].update(kind="glu")))
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(broken(lambda r: r["layers"][3]["mixer"].update(kv_from=5)))
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(broken(lambda r: r["layers"][3]["mixer"].update(kv_from=1)))
    with pytest.raises(ConfigError, match="differ"):
        config_from_dict(broken(lambda r: r["layers"][3]["mixer"].update(vdim=16)))
    with pytest.raises(ConfigError, match="diff"):
        config_from_dict(broken(lambda r: r["layers"][0]["mixer"].update(diff=1.5)))
    with pytest.raises(ConfigError, match="norm"):
        config_from_dict(broken(lambda r: r.pop("norm")))
    with pytest.raises(ConfigError, match="streams"):
        config_from_dict(broken(lambda r: r.update(streams=0)))


# ------------------------------------------------------------------ the plain mechanisms against closed forms
def test_convolution_is_causal_and_starts_from_zeros():
    u, w = torch.randn(9, 3, dtype=F64), torch.randn(3, 4, dtype=F64)
    y = P.causal_conv(u, w)
    assert torch.allclose(y[0], w[:, 3] * u[0])
    assert torch.allclose(y[5], sum(w[:, j] * u[5 - 3 + j] for j in range(4)))
    u2 = u.clone()
    u2[6:] += 1.0
    assert torch.allclose(P.causal_conv(u2, w)[:6], y[:6])


def test_both_rotations_leave_the_rest_and_keep_lengths():
    x = torch.randn(6, 2, 10, dtype=F64)
    p, i = 4, 1
    a = p * 100.0 ** (-2 * i / 6)
    y = P.rotate_neighbours(x, 100.0, 6)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., :6].pow(2).sum(-1), x[..., :6].pow(2).sum(-1))
    assert torch.allclose(y[p, 0, 2], x[p, 0, 2] * math.cos(a) - x[p, 0, 3] * math.sin(a))
    assert torch.allclose(y[p, 0, 3], x[p, 0, 3] * math.cos(a) + x[p, 0, 2] * math.sin(a))
    y = P.rotate_halves(x, 100.0, 6)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[p, 1, 1], x[p, 1, 1] * math.cos(a) - x[p, 1, 4] * math.sin(a))
    assert torch.allclose(y[p, 1, 4], x[p, 1, 4] * math.cos(a) + x[p, 1, 1] * math.sin(a))


def test_a_window_holds_the_row_itself_and_the_tokens_before_it():
    see = P.visible(10, 4)
    assert see[2].tolist() == [True] * 3 + [False] * 7
    assert see[9].tolist() == [False] * 6 + [True] * 4
    assert P.visible(5)[4].tolist() == [True] * 5


def test_differential_attention_of_equal_maps_is_one_map_normed():
    """With both maps' queries and keys equal, a head is ``(1 - lambda) a``, and the unit norm leaves ``a / rms(a)`` with
    the sign of ``1 - lambda``, times ``1 - diff``; a gate projection of zeros halves it."""
    torch.manual_seed(0)
    n, w, d, dv, diff = 7, 12, 4, 6, 0.3
    m = {"heads": 1, "kv_heads": 1, "dim": d, "vdim": dv, "scale": 0.5, "diff": diff}
    qw, kw = torch.randn(d, w, dtype=F64), torch.randn(d, w, dtype=F64)
    t = {"q": torch.cat([qw, qw]), "q.b": torch.zeros(2 * d, dtype=F64), "k": torch.cat([kw, kw]), "k.b": torch.zeros(2 * d, dtype=F64),
         "v": torch.randn(dv, w, dtype=F64), "v.b": torch.randn(dv, dtype=F64), "g": torch.zeros(dv, w, dtype=F64), "o": torch.eye(dv, dtype=F64),
         "o.b": torch.zeros(dv, dtype=F64), "lq1": torch.full((d,), 0.5, dtype=F64), "lk1": torch.ones(d, dtype=F64),
         "lq2": torch.zeros(d, dtype=F64), "lk2": torch.zeros(d, dtype=F64)}
    h = torch.randn(n, w, dtype=F64)
    lam = math.exp(2.0) - 1.0 + diff
    assert torch.allclose(P.diff_lambda(t, "", diff, F64), torch.tensor(lam, dtype=F64))
    got, _ = P.diff_attention(t, "", m, h, 1e-12)
    a = P.softmax_rows((h @ qw.T) @ (h @ kw.T).T * 0.5, P.visible(n)) @ (h @ t["v"].T + t["v.b"])
    assert torch.allclose(got, -P.rms(a, 1e-12) * (1 - diff) * 0.5, atol=1e-9)


def test_state_space_layer_in_closed_form_for_constant_inputs():
    """One head, one state, one tap: with constant x, B, C and step size, ``y_n = C B dt x sum_(j<=n) a^(n-j) + D x``."""
    n, w = 6, 3
    m = {"heads": 1, "vdim": 2, "state": 1, "groups": 1, "conv": 1, "norm_groups": 1}
    # rows of `in`: z (2), x (2), B, C, dt; the input is the same for every token
    win = torch.zeros(7, w, dtype=F64)
    win[0:2, 0] = 50.0           # silu(z) = z: the gate multiplies by 50
    win[2, 1], win[3, 1] = 1.0, 2.0
    win[4, 2], win[5, 2], win[6, 2] = 1.0, 3.0, 0.7
    t = {"in": win, "conv": torch.ones(4, 1, dtype=F64), "conv.b": torch.zeros(4, dtype=F64), "dt_bias": torch.tensor([0.1], dtype=F64),
         "A_log": torch.tensor([0.3], dtype=F64), "D": torch.tensor([0.9], dtype=F64), "norm": torch.ones(2, dtype=F64), "o": torch.eye(2, dtype=F64)}
    h = torch.ones(n, w, dtype=F64)
    sl = lambda v: v / (1 + math.exp(-v))
    x, B, C = torch.tensor([sl(1.0), sl(2.0)], dtype=F64), sl(1.0), sl(3.0)
    dt = math.log1p(math.exp(0.8))
    a = math.exp(-math.exp(0.3) * dt)
    got = P.mamba2(t, "", m, h, 0.0)
    for i in range(n):
        y = (C * B * dt * sum(a ** (i - j) for j in range(i + 1)) + 0.9) * x * 50.0
        assert torch.allclose(got[i], y / torch.sqrt((y * y).mean()), atol=1e-9)


def test_the_correction_changes_the_choice_and_not_the_weights():
    t = {"router": torch.eye(4, dtype=F64), "correction": torch.tensor([0.0, 0.0, 0.0, 1.0], dtype=F64)}
    mlp = {"router": {"experts": 4, "top": 2, "identity": 0}}
    h = torch.tensor([[3.0, 1.0, 2.0, -9.0]], dtype=F64)
    chosen, w = P.route(t, "", mlp, h)
    s = torch.softmax(h[0], 0)
    assert sorted(chosen[0].tolist()) == [0, 3]          # without the correction: 0 and 2
    want = {0: s[0] / (s[0] + s[3]), 3: s[3] / (s[0] + s[3])}
    for e, g in zip(chosen[0].tolist(), w[0]):
        assert torch.allclose(g, want[e])


def test_identity_experts_return_their_input():
    w_ = 4
    t = {"router": torch.tensor([[0.0] * w_, [5.0, 0, 0, 0]], dtype=F64), "correction": torch.zeros(2, dtype=F64),
         "e0.gate": torch.randn(3, w_, dtype=F64), "e0.up": torch.randn(3, w_, dtype=F64), "e0.down": torch.randn(w_, 3, dtype=F64)}
    mlp = {"router": {"experts": 1, "top": 1, "identity": 1}, "expert": {"ff": 3}}
    h = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-1.0, 0.5, 0.0, 2.0]], dtype=F64)
    out = P.moe(t, "", mlp, h)
    assert torch.allclose(out[0], h[0])                                     # the identity expert alone: weight one
    assert torch.allclose(out[1], P.expert(t, "", 0, h[1:2])[0])            # the real expert alone


def test_streams_are_mixed_from_to():
    t = {"in": torch.tensor([2.0, -1.0], dtype=F64), "out": torch.tensor([0.5, 3.0], dtype=F64), "mix": torch.tensor([[1.0, 10.0], [100.0, 1000.0]], dtype=F64)}
    xs = torch.stack([torch.full((1, 2), 1.0, dtype=F64), torch.full((1, 2), 2.0, dtype=F64)])
    assert torch.allclose(P.streams_read(t, "", xs), torch.zeros(1, 2, dtype=F64))
    new = P.streams_write(t, "", xs, torch.ones(1, 2, dtype=F64))
    assert torch.allclose(new[0], torch.full((1, 2), 1.0 + 200.0 + 0.5, dtype=F64)) and torch.allclose(new[1], torch.full((1, 2), 10.0 + 2000.0 + 3.0, dtype=F64))


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
    n = 70 if name != "wide" else 40
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
    """The convolutions' last inputs and the state-space layers' states belong to the slot."""
    d = U.make_dir(tmp_path, "odd", seed=5)
    lm = loaded(d, max_requests=1)
    a, b = U.tokens_of(9, 61, 1), U.tokens_of(6, 61, 2)
    U.run_schedule(lm, {"a": a}, [[("a", 9)]])
    got = U.run_schedule(lm, {"b": b}, [[("b", 2)], [("b", 4)]])["b"]
    assert U.relative_error(got, U.plain_logits(d, b)) < TOL


def test_what_the_layers_ask_of_the_cache(tmp_path):
    lm = loaded(U.make_dir(tmp_path, "mixed", seed=6))
    # the two attention layers share one cache of all keys (four key maps, heads filled up to the attention tile); one
    # latent layer sees a window, the other everything, each as one head
    groups = {name: (g.spec.window, g.spec.kv_heads) for name, g in lm.cache.groups.items()}
    assert sorted(groups.values(), key=str) == sorted([(None, 4), (20, 1), (None, 1)], key=str)
    states = lm.cache.states
    assert states[(0, 1)].shapes == {"conv": (2, 2 * 4 * 16 + 2 * 2 * 16 + 2 * 2 * 24)}   # q, k and v (a value head once per map) before the taps
    assert states[(3, 1)].shapes == {"conv": (1, 2 * 4 * 16)}                             # the layer that reads layer 0's cache: its queries
    assert lm.cache.shared[(3, 0)] == 0
    assert states[(1, 0)].shapes == {"conv": (2, 4 * 16 + 2 * 2 * 8), "ssm": (4, 8, 16)}
    assert (2, 0) not in states and (5, 0) not in states


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


def test_a_layer_without_feed_forward_may_bring_its_unused_tensors(tmp_path):
    """The second norm and the second streams' tensors of a layer that has no feed-forward are not used and not missed;
    any other tensor the model does not know is still refused by name."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights.loader import WeightsError
    d = U.make_dir(tmp_path, "mixed", seed=8)
    path = d + "/model.safetensors"
    w = load_file(path)
    w.update({"l2.norm2": torch.ones(64), "l2.hc2.in": torch.ones(3), "l2.hc2.out": torch.ones(3), "l2.hc2.mix": torch.eye(3)})
    save_file(w, path)
    toks = U.tokens_of(9, 97, 1)
    got = U.run_schedule(loaded(d), {"a": toks}, [[("a", 9)]])["a"]
    assert U.relative_error(got, U.plain_logits(d, toks)) < TOL
    w["l2.mlp.router"] = torch.ones(3, 64)
    save_file(w, path)
    with pytest.raises(WeightsError, match="l2.mlp.router"):
        loaded(d)
