"""Befirax on the GPU: every new kernel alone against the CPU stand-in of the same entry point (written from the
mechanisms' equations) or the plain model's function, and the whole engine (cuts of prompts, decoding, mixed batches with
pages and slots used again, captured steps, generation) against the plain model."""
import pytest
import torch

import befirax_util as U
from emulated_ops import EmulatedOps
from gpu_util import DEV
from plain import befirax_plain as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
F32 = 1e-4     # float32 against the plain model in 64-bit
F64 = torch.float64


def sharpen_for(dtype):
    """Softmaxes far from flat for the 32-bit runs, where a wrong key must show; milder for bfloat16, whose rounding a
    sharp softmax multiplies."""
    return 6.0 if dtype == torch.float32 else 2.5


def ops_of(dtype):
    from machserve_amd.kernels import get_ops
    return get_ops(dtype, DEV)


def dev(t, dtype=None):
    return None if t is None else t.to(device=DEV, dtype=dtype or t.dtype).contiguous()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def close(got, want, dtype, what="", scale_by=None):
    got, want = got.float().cpu().double(), want.double().cpu()
    bound = (1e-4 if dtype == torch.float32 else 2e-2) * float((scale_by if scale_by is not None else want).abs().max()) + 1e-6
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: error {err:.3e} over {bound:.3e}"


def _steps(lens, cuts):
    """Three requests' rows in steps: each step takes a request's next ``cuts[s]`` rows.  Yields (rows, first row of each
    request in the step, rows of each, slots)."""
    starts = [sum(lens[:s]) for s in range(len(lens))]
    at = [0] * len(lens)
    while any(a < n for a, n in zip(at, lens)):
        rows, q0, ql, slots = [], [], [], []
        for s in range(len(lens)):
            c = min(cuts[s], lens[s] - at[s])
            if c > 0:
                q0.append(len(rows)); ql.append(c); slots.append(s + 1)
                rows += list(range(starts[s] + at[s], starts[s] + at[s] + c))
                at[s] += c
        yield rows, q0, ql, slots


# ------------------------------------------------------------------ several residual streams
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S,d,T", [(1, 48, 5), (2, 130, 37), (3, 1024, 70), (8, 64, 3)])
def test_streams_read_and_written(dtype, S, d, T):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(S * d)
    xs, w_in, nw = torch.randn(S, T, d), torch.randn(S), torch.randn(d)
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    close(ops.streams_read(dev(xs), dev(w_in)), ref.streams_read(xs, w_in), torch.float32, "weighted sum")
    close(ops.streams_read(dev(xs), None, dev(rows)), ref.streams_read(xs, None, rows), torch.float32, "plain sum of chosen rows")
    close(ops.streams_read_norm(dev(xs), dev(w_in), dev(nw), 1e-5), ref.streams_read_norm(xs, w_in, nw, 1e-5), dtype, "sum and norm")
    for parts, bias in ((1, None), (3, torch.randn(d))):
        sums, mix, w_out = torch.randn(parts, T, d), torch.randn(S, S), torch.randn(S)
        want = xs.clone()
        ref.streams_write(want, sums, bias, mix, w_out)
        got = dev(xs)
        ops.streams_write(got, dev(sums), dev(bias), dev(mix), dev(w_out))
        close(got, want, torch.float32, f"all streams at once from {parts} sums")
        both = dev(xs)
        h = ops.streams_write_read_norm(both, dev(sums), dev(bias), dev(mix), dev(w_out), dev(w_in), dev(nw), 1e-5)
        close(both, want, torch.float32, "a write with the next read in its kernel leaves the same streams")
        close(h, ref.streams_read_norm(want, w_in, nw, 1e-5), dtype, "and the same input of the next branch")


def test_streams_beyond_the_kernels_are_refused():
    ops = ops_of(torch.float32)
    from machserve_amd.kernels.ops import KernelError
    with pytest.raises(KernelError, match="streams"):
        ops.streams_read(torch.zeros(ops.streams_limits()["streams"] + 1, 2, 8, device=DEV), None)


# ------------------------------------------------------------------ routed experts with gates, corrected choice, identity experts
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,ff,identity,width", [(6, 2, 24, 1, 64), (3, 3, 8, 0, 48), (7, 1, 24, 3, 48), (32, 4, 32, 4, 128), (5, 3, 12, 2, 40),
                                                     (2, 4, 8, 2, 64), (66, 64, 8, 4, 64)])
def test_gated_experts_with_corrected_choice_against_the_plain_feed_forward(dtype, E, top, ff, identity, width):
    ops = ops_of(dtype)
    torch.manual_seed(E * ff + identity)
    T = 37
    h = torch.randn(T, width).to(dtype)
    t = {"router": torch.randn(E + identity, width) * 0.3, "correction": torch.randn(E + identity) * 0.2}
    for e in range(E):
        for s in ("gate", "up"):
            t[f"e{e}.{s}"] = (torch.randn(ff, width) * width ** -0.5).to(dtype).float()
        t[f"e{e}.down"] = (torch.randn(width, ff) * ff ** -0.5).to(dtype).float()
    mlp = {"router": {"experts": E, "top": top, "identity": identity}, "expert": {"ff": ff}}
    t64 = {k: v.double() for k, v in t.items()}
    want = P.moe(t64, "", mlp, h.double())
    idx, wts = P.route(t64, "", mlp, h.double())
    gates = ops.route(dev(h), dev(t["router"]), None, top, correction=dev(t["correction"]), softmax_all=True)
    close(gates, torch.zeros(T, E + identity, dtype=F64).scatter_(1, idx, wts), torch.float32, "weights of the chosen outputs, zero elsewhere")
    fill = -(E * ff) % 8
    zeros = [torch.zeros(fill, width)] if fill else []
    w_up = torch.cat([t[f"e{e}.gate"] for e in range(E)] + zeros + [t[f"e{e}.up"] for e in range(E)] + zeros)
    w_down = torch.cat([t[f"e{e}.down"] for e in range(E)] + ([torch.zeros(width, fill)] if fill else []), 1)
    a = ops.expert_act(ops.linear(dev(h), dev(w_up, dtype), None, out_f32=True), gates, ff, "silu", experts=E, gated=True)
    got = ops.linear(a, dev(w_down, dtype), None, out_f32=True)
    if identity:
        ops.add_scaled_rows(got, dev(h), gates, E, identity)
    close(got, want, dtype, "the weighted sum of the chosen experts and the input's rows")


def test_the_router_without_correction_weighs_the_largest_scores():
    ops = ops_of(torch.float32)
    h, w = torch.eye(4), torch.tensor([[3.0, 1.0, 2.0, -9.0]]).t().contiguous().expand(4, 4).contiguous()
    gates = ops.route(dev(h[:1]), dev(torch.diag(torch.tensor([3.0, 1.0, 2.0, -9.0]))[:, :4].contiguous() + 0 * w), None, 2, softmax_all=True).cpu()
    s = torch.softmax(torch.tensor([3.0, 0.0, 0.0, 0.0]), 0)
    assert gates[0, 0] > 0 and (gates[0] > 0).sum() == 2 and abs(float(gates[0].sum()) - 1.0) < 1e-6
    assert abs(float(gates[0, 0]) - float(s[0] / (s[0] + s[1]))) < 1e-6


# ------------------------------------------------------------------ the state-space layer
def _ssd_case(dtype, H, P_, N, G, parts, lens, cuts_list):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(H * P_ + N)
    T, inner = sum(lens), H * P_
    C = inner + 2 * G * N
    ld = 2 * inner + 2 * G * N + H
    proj = torch.randn(T, ld)
    proj[:, inner + C:] -= 2.0  # small steps: the state lives long
    xbc = torch.randn(T, C)
    dt_bias, a_log, d_skip, nw = torch.randn(H) * 0.3, torch.randn(H) * 0.5, torch.randn(H), torch.randn(inner)
    out_cols = -(-inner // 8) * 8
    want_state = torch.zeros(5, H, N, P_)
    whole = list(_steps(lens, lens))
    assert len(whole) == 1
    rows, q0, ql, slots = whole[0]
    y = ref.ssd_scan(xbc, proj, inner + C, dt_bias, a_log, d_skip, want_state, torch.tensor(q0), torch.tensor(ql), torch.tensor(slots), H, P_, N, G)
    want = ref.gated_group_norm(y, proj, 0, nw, 1e-5, parts, out_cols)
    for cuts in cuts_list:
        state = torch.zeros(5, H, N, P_, device=DEV)
        got_y, got = torch.zeros(T, inner), torch.zeros(T, out_cols)
        for rows, q0, ql, slots in _steps(lens, cuts):
            r = torch.tensor(rows)
            yy = ops.ssd_scan(dev(xbc[r]), dev(proj[r]), inner + C, dev(dt_bias), dev(a_log), dev(d_skip), state, i32(q0), i32(ql), i32(slots), H, P_, N, G)
            got_y[r] = yy.cpu()
            got[r] = ops.gated_group_norm(yy, dev(proj[r]), 0, dev(nw), 1e-5, parts, out_cols).float().cpu()
        close(got_y, y, torch.float32, f"recurrence in steps of {cuts}")
        close(state.cpu(), want_state, torch.float32, f"state after steps of {cuts}")
        close(got, want, dtype, f"gated norm in {parts} parts")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,P_,N,G,parts", [(4, 16, 8, 2, 2), (3, 8, 5, 3, 3), (2, 64, 64, 1, 1), (2, 32, 16, 1, 4), (6, 48, 128, 2, 2), (1, 100, 33, 1, 5),
                                            (8, 64, 130, 4, 1)])
def test_state_space_recurrence_in_one_step_and_in_many(dtype, H, P_, N, G, parts):
    _ssd_case(dtype, H, P_, N, G, parts, [23, 1, 40], [[23, 1, 40], [1, 1, 1], [7, 1, 9], [2, 1, 64]])


def test_state_space_recurrence_of_a_long_prompt():
    """Prompts long enough for segments of the usual length, whole and in portions, beside a short request."""
    _ssd_case(torch.float32, 4, 32, 16, 2, 2, [700, 3, 333], [[700, 3, 333], [300, 1, 170]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,P_,N,G,seg", [(4, 16, 8, 2, 8), (3, 8, 5, 3, 5), (2, 64, 64, 1, 16), (2, 100, 130, 2, 3)])
def test_state_space_recurrence_walked_in_segments(monkeypatch, dtype, H, P_, N, G, seg):
    """Requests of unequal lengths whose rows are walked in short segments side by side: a request of one segment, one that
    ends on a segment's edge, one that ends just behind an edge; first whole, then in portions that start from a state."""
    ops = ops_of(dtype)
    monkeypatch.setattr(type(ops), "SCAN_CHUNK_MIN_ROWS", 2 * seg)
    monkeypatch.setattr(type(ops), "SSD_SEGMENT", seg)
    lens = [4 * seg, 3, 9 * seg + 1]
    _ssd_case(dtype, H, P_, N, G, 1, lens, ([1000, 1000, 1000], [3 * seg - 1, 2, 4 * seg + 2], [2 * seg, 1, 2 * seg]))


def test_sizes_the_state_space_kernels_do_not_take_are_refused_when_the_part_is_built():
    from machserve_amd.config import StateSpaceDualSpec
    from machserve_amd.parts import MIXERS, Runtime
    rt = Runtime(torch.device(DEV), torch.bfloat16, ops_of(torch.bfloat16))
    lim = rt.ops.ssd_limits()
    MIXERS.build(StateSpaceDualSpec("mamba2", 64, 2, lim["head_dim"], lim["states"], 1, 4), rt)
    with pytest.raises(ValueError, match="states"):
        MIXERS.build(StateSpaceDualSpec("mamba2", 64, 2, 16, lim["states"] + 1, 1, 4), rt)


# ------------------------------------------------------------------ differential attention
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,dv", [(4, 2, 32, 24), (6, 1, 32, 10), (2, 2, 16, 8), (2, 2, 64, 64), (8, 2, 128, 128), (5, 5, 96, 70)])
def test_two_maps_combined_normed_and_gated(dtype, H, KV, hd, dv):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(H * hd)
    T, cols = 19, -(-H * dv // 8) * 8
    o, gate = torch.randn(T, 2 * H * hd).to(dtype), torch.randn(T, H * dv)
    for lam in (0.7, -1.3):
        close(ops.diff_combine(dev(o), dev(gate), lam, 1e-6, 0.75, H, KV, hd, dv, cols), ref.diff_combine(o, gate, lam, 1e-6, 0.75, H, KV, hd, dv, cols),
              dtype, f"lambda {lam}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,dv,rot", [(8, 4, 16, 24, 8), (12, 2, 20, 10, 0), (4, 4, 64, 64, 32)])
def test_rows_of_queries_alone_finished(dtype, H, KV, d, dv, rot):
    """A layer that reads another layer's keys and values finishes its queries and leaves the pools as they are."""
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(d)
    T, ps, dp = 21, 16, -(-max(d, dv) // 16) * 16
    rows, pos = torch.randn(T, H * d), torch.randint(0, 500, (T,), dtype=torch.int32)
    inv = (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float32) * 2 / rot)) if rot else None
    slots = torch.arange(T, dtype=torch.int32) + ps
    kpool, vpool = torch.randn(4, KV, ps, dp).to(dtype), torch.randn(4, KV, dp, ps).to(dtype)
    want = ref.finish_rows(rows, None, None, 1e-6, pos, inv, rot, True, slots, kpool.clone(), vpool.clone(), H, KV, d, dv, ps, queries_only=True)
    gk, gv = dev(kpool), dev(vpool)
    got = ops.finish_rows(dev(rows), None, None, 1e-6, dev(pos), dev(inv), rot, True, dev(slots), gk, gv, H, KV, d, dv, ps, queries_only=True)
    close(got, want, dtype, "queries")
    assert torch.equal(gk.cpu(), kpool) and torch.equal(gv.cpu(), vpool)


# ------------------------------------------------------------------ attention through a latent: halves, direct queries, gate
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,rot,rank", [(3, 16, 8, 24), (5, 8, 6, 20), (17, 16, 16, 48), (2, 64, 32, 96)])
def test_latent_rows_and_queries_rotated_half_against_half(dtype, H, d, rot, rank):
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(rank)
    T, ps, hd = 13, 16, -(-(rank + rot) // 16) * 16
    pos = torch.randint(0, 900, (T,), dtype=torch.int32)
    inv = 1000.0 ** (-torch.arange(rot // 2, dtype=torch.float32) * 2 / rot)
    slots = torch.randperm(3 * ps)[:T].int() + ps
    proj, cn = torch.randn(2, T, rank + rot), torch.randn(rank)
    kpool, vpool = torch.zeros(5, 1, ps, hd).to(dtype), torch.zeros(5, 1, hd, ps).to(dtype)
    assert ref.latent_rows(proj, None, cn, 1e-6, pos, inv, 1.0, slots, kpool, vpool, 0, rank, rot, ps, halves=True) is None
    gk, gv = torch.zeros(5, 1, ps, hd, dtype=dtype, device=DEV), torch.zeros(5, 1, hd, ps, dtype=dtype, device=DEV)
    assert ops.latent_rows(dev(proj), None, dev(cn), 1e-6, dev(pos), dev(inv), 1.0, dev(slots), gk, gv, 0, rank, rot, ps, halves=True) is None
    close(gk, kpool, dtype, "latent and key part in the pages")
    close(gv, vpool, dtype, "latent as the value")
    q = torch.randn(T, H * (d + rot))
    (wp, wa), (gp, ga) = ref.latent_query(q, pos, inv, 1.0, H, d, rot, rank, hd, halves=True), ops.latent_query(dev(q), dev(pos), dev(inv), 1.0, H, d, rot, rank, hd, halves=True)
    close(gp, wp, dtype, "plain parts")
    close(ga[..., rank:], wa[..., rank:], dtype, "rotated parts behind the latent's columns")
    g = torch.randn(T, H)
    close(ops.sigmoid_rows(dev(g)), torch.sigmoid(g), torch.float32, "gates")


def _keys_case(dtype, H, KV, hd, ps, before, now, key, window, gate=None):
    """One request with ``before`` keys in the cache and ``now`` rows; key ``key`` is made to stand out for the last row's
    first head of every group (its value is 50 in every column).  The kernels against the stand-in; returns the last row."""
    ops, ref = ops_of(dtype), EmulatedOps(dtype)
    torch.manual_seed(before + now)
    total = before + now
    n_pages = -(-total // ps)
    table = (torch.randperm(n_pages) + 1).int().view(1, -1)
    kpool, vpool = torch.randn(n_pages + 1, KV, ps, hd).to(dtype), torch.randn(n_pages + 1, KV, hd, ps).to(dtype)
    q = torch.randn(now, H * hd)
    page, off = int(table[0, key // ps]), key % ps
    for kvh in range(KV):
        h = kvh * (H // KV)
        kpool[page, kvh, off] = (q[-1, h * hd:(h + 1) * hd] * 4).to(dtype)
    vpool[page, :, :, off] = 50.0
    q = q.to(dtype)
    g = H // KV
    unit = ops.attention_rows_per_block(hd)
    ref.rows_per_block = unit
    work = torch.tensor([[0, r0] for r0 in range(0, now * g, unit)], dtype=torch.int32)
    args = (torch.tensor([0], dtype=torch.int32), torch.tensor([now], dtype=torch.int32), torch.tensor([before], dtype=torch.int32))
    want = ref.paged_attention(q, kpool, vpool, table, *args, work, H, KV, hd, ps, window, 0.5, out_gate=gate)
    got = ops.paged_attention(dev(q), dev(kpool), dev(vpool), dev(table), *[dev(a) for a in args], dev(work), H, KV, hd, ps, window, 0.5, out_gate=dev(gate))
    close(got[-1:], want[-1:], dtype, "mixed-batch kernel", scale_by=want.abs().max().clamp(min=1.0))
    if now == 1 and g <= ops.DECODE_MAX_GROUP:
        got = ops.decode_attention(dev(q), dev(kpool), dev(vpool), dev(table), dev(args[2]), H, KV, hd, ps, window, 0.5, None, dev(gate))
        close(got, want, dtype, "decode kernel", scale_by=want.abs().max().clamp(min=1.0))
    return want[-1]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("window,n,key,seen", [(136, 800, 664, True), (136, 800, 663, False), (136, 800, 799, True), (20, 300, 280, True), (20, 300, 279, False),
                                               (64, 640, 576, True), (64, 640, 575, False), (7, 50, 43, True), (7, 50, 42, False), (1000, 800, 0, True),
                                               (200, 200, 0, True), (200, 201, 0, False), (200, 201, 1, True), (None, 800, 0, True), (None, 800, 511, True)])
def test_a_key_that_stands_out_is_seen_only_inside_the_window(dtype, decoded, window, n, key, seen):
    """The last row of ``n`` over one latent head shared by six query heads, with a gate per head: the first key the window
    still holds and the one before it, keys at page borders, the first key of all, the row itself."""
    gate = torch.full((1 if decoded else n, 6), 0.5)
    last = _keys_case(dtype, 6, 1, 96, 16, n - 1 if decoded else 0, 1 if decoded else n, key, window, gate)
    top = float(last[:96].min())
    assert (20.0 < top < 30.0) if seen else top < 10.0   # 50, halved by the gate


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("n,key", [(900, 0), (900, 3), (900, 447), (900, 448), (900, 899), (65, 0)])
def test_a_far_key_in_one_map_shows_in_the_heads_result(dtype, decoded, n, key):
    """Two heads over one key/value head, as four maps over two key heads: the key stands out for the first map of each
    key head, whose heads then come out as plus ``factor`` in every column, whatever the other keys hold."""
    H, KV, hd, dv = 2, 1, 32, 32
    last = _keys_case(dtype, 2 * H, 2 * KV, hd, 16, n - 1 if decoded else 0, 1 if decoded else n, key, None)
    ops = ops_of(dtype)
    y = ops.diff_combine(dev(last.view(1, -1).to(dtype)), torch.zeros(1, H * dv, device=DEV), 0.8, 1e-6, 0.7, H, KV, hd, dv, H * dv).float().cpu()[0]
    # maps in the order (key head, map, head of the group): the first query map of key head 0 is head 0's first map,
    # that of key head 1 (the second map of the key/value head) is head 0's second map
    assert float((y[:dv] - 0.35 * (1 - 0.8) / abs(1 - 0.8)).abs().max()) < 0.05


# ------------------------------------------------------------------ the engine against the plain model
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
def test_sizes_nearer_a_real_models(tmp_path, dtype):
    # in bfloat16 the experts stay small beside the stream: with sixteen experts and hundreds of rows some row's choice
    # sits on a near-tie, and the rows behind it inherit what it does to the recurrences' states
    d = U.make_dir(tmp_path, "big", seed=17, sharpen=2.0, experts=8.0 if dtype == torch.float32 else 1.0)
    n = 330
    toks = U.tokens_of(n, 1000, 4)
    want = plain_for(d, dtype, toks)
    lm = loaded(d, dtype, page_size=64)
    for what, schedule in {"whole": [[("a", n)]], "portions, then token by token": _cut("a", 290, [128, 2, 97, 63]) + [[("a", 1)]] * 40}.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.within(got, want, dtype), what


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
@pytest.mark.parametrize("name", ["odd", "wide"])
def test_long_decoding_from_captured_steps(tmp_path, name, dtype):
    """Decoded tokens pass every window of the configurations (7 and 200 positions) and leave pages behind."""
    d = U.make_dir(tmp_path, name, seed=10, sharpen=sharpen_for(dtype))
    toks = U.tokens_of(330, U.CONFIGS[name]["vocab"], 3)
    lm = loaded(d, dtype, max_tokens=512)
    got = U.run_schedule(lm, {"a": toks}, [[("a", 10)]] + [[("a", 1)]] * 320)["a"]
    assert U.within(got, plain_for(d, dtype, toks), dtype)
    assert len(lm.step._graphs) > 0     # the single rows ran from captured steps


def test_a_long_prompt_in_portions_behind_pages_of_64(tmp_path):
    """A recurrence over a thousand tokens and windows across many pages, in a step of many rows and in portions that end
    inside pages and windows."""
    d = U.make_dir(tmp_path, "mixed", seed=11)
    toks = U.tokens_of(1100, 97, 6)
    want = plain_for(d, torch.float32, toks)
    lm = loaded(d, torch.float32, page_size=64, max_tokens=1152)
    for what, schedule in {"whole": [[("a", 1100)]], "portions": _cut("a", 1100, [500, 63, 2, 129, 300, 7])}.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.relative_error(got, want) < F32, what


def test_long_portions_beside_decoded_tokens(tmp_path):
    d = U.make_dir(tmp_path, "mixed", seed=21)
    reqs = {"a": U.tokens_of(700, 97, 1), "b": U.tokens_of(420, 97, 2), "c": U.tokens_of(9, 97, 3)}
    schedule = [[("a", 290), ("b", 300)], [("c", 7), ("b", 118)], [("b", 1), ("a", 405), ("c", 1)], [("b", 1), ("a", 5), ("c", 1)]]
    lm = loaded(d, torch.float32, page_size=64, max_tokens=1344, max_requests=3)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.relative_error(got[i], plain_for(d, torch.float32, toks)) < F32, i


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


def test_a_window_one_token_off_or_a_state_lost_would_show(tmp_path):
    """The tests' own power: the plain model with every window one token longer is far from the engine, and so is the
    engine with its slot's states zeroed half way."""
    import json
    import os
    d = U.make_dir(tmp_path, "mixed", seed=16)
    toks = U.tokens_of(60, 97, 9)
    want = plain_for(d, torch.float32, toks)
    w, cfg = U.read(d)
    off = json.loads(json.dumps(cfg))
    for layer in off["layers"]:
        if "mask" in layer["mixer"]:
            layer["mixer"]["mask"]["size"] += 1
    assert U.relative_error(P.forward(w, off, toks, torch.float64)[30:], want[30:]) > 3e-3   # one layer of six sees a window
    lm = loaded(d, torch.float32, use_graphs=False)
    from machserve_amd.engine.step import StepEntry
    slot = lm.cache.admit()
    lm.step([StepEntry(slot, toks[:30], [])])
    lm.device_cache.zero_state(slot)
    got = lm.step([StepEntry(slot, toks[30:], list(range(30)))]).float().cpu()
    lm.cache.release(slot)
    assert U.relative_error(got, want[30:]) > 1e-2
    assert os.path.isdir(d)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, dtype):
    import machserve_amd
    d = U.make_dir(tmp_path, "mixed", seed=13, sharpen=3.0)
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
    d = U.make_dir(tmp_path, "mixed", seed=15)
    w, cfg = U.read(d)
    prompt = U.tokens_of(9, 97, 4)
    cmd = [sys.executable, os.path.join(root, "bin", "machserve"), "--max-new", "5", "--dtype", "f32", "--tpp", "16", "--prompt-ids"]
    r = subprocess.run(cmd + [",".join(map(str, prompt)), "--model", d], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.split()] == P.greedy_generate(w, cfg, prompt, 5, torch.float64)
