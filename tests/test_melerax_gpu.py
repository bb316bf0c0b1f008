"""Melerax on the GPU: every new kernel alone against the CPU stand-in of the same entry point (written from the
mechanisms' equations) or the plain model's function, and the whole engine (cuts of prompts, decoding, mixed batches with
pages and slots used again, captured steps, generation) against the plain model."""
import pytest
import torch

import melerax_util as U
from emulated_ops import EmulatedOps
from gpu_util import DEV
from plain import melerax_plain as P

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
    request in the step, rows of each, slots, positions of the rows)."""
    starts = [sum(lens[:s]) for s in range(len(lens))]
    at = [0] * len(lens)
    while any(a < n for a, n in zip(at, lens)):
        rows, q0, ql, slots, pos = [], [], [], [], []
        for s in range(len(lens)):
            c = min(cuts[s], lens[s] - at[s])
            if c > 0:
                q0.append(len(rows)); ql.append(c); slots.append(s + 1)
                rows += list(range(starts[s] + at[s], starts[s] + at[s] + c))
                pos += list(range(at[s], at[s] + c))
                at[s] += c
        yield rows, q0, ql, slots, pos


CUTS = ([1000, 1000, 1000], [1, 1, 1], [2, 1, 5], [64, 1, 29])


# ------------------------------------------------------------------ kernels, each alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_of_pairs_in_one_step_and_in_many(dtype):
    ops = ops_of(dtype)
    V, d, buckets = 50, 24, 11
    torch.manual_seed(0)
    table, pairs = torch.randn(V, d).to(dtype), torch.randn(buckets + 1, d).to(dtype)
    lens = [9, 1, 30]
    toks = torch.randint(0, V, (sum(lens),))
    starts = [0, 9, 10]
    want = torch.cat([table[toks[s:s + n]].double() + pairs[torch.as_tensor(P.bigram_rows(toks[s:s + n].tolist(), 7, 3, buckets)).long()].double()
                      for s, n in zip(starts, lens)])
    for cuts in CUTS:
        prev = torch.zeros(5, dtype=torch.int32, device=DEV)
        got = torch.zeros(sum(lens), d)
        for rows, q0, ql, slots, pos in _steps(lens, cuts):
            p0 = [pos[q] for q in q0]
            got[rows] = ops.embed_pair(dev(toks[rows].int()), dev(table), dev(pairs), prev, i32(q0), i32(ql), i32(p0), i32(slots), 7, 3, buckets).cpu()
        close(got, want, torch.float32, f"steps of {cuts}")


@pytest.mark.parametrize("C,taps,biases", [(40, 1, True), (48, 2, False), (300, 4, True), (24, 16, True)])
def test_convolution_over_sums_in_one_step_and_in_many(C, taps, biases):
    ops = ops_of(torch.float32)
    torch.manual_seed(C)
    lens = [11, 1, 75]
    sums = torch.randn(2, sum(lens), C + 16)
    w, b_in, b_out = torch.randn(C, taps) * 0.5, (torch.randn(C) if biases else None), (torch.randn(C) if biases else None)
    u = sums.sum(0)[:, 8:8 + C].double() + (b_in.double() if biases else 0.0)
    want = torch.cat([P.causal_conv(u[s:s + n], w.double()) for s, n in zip([0, 11, 12], lens)]) + (b_out.double() if biases else 0.0)
    for cuts in CUTS:
        state = torch.zeros(5, taps - 1, C, device=DEV) if taps > 1 else None
        got = torch.zeros(sum(lens), C)
        for rows, q0, ql, slots, _ in _steps(lens, cuts):
            got[rows] = ops.conv_sums(dev(sums[:, rows]), 8, C, dev(b_in), dev(w), dev(b_out), state, i32(q0), i32(ql), i32(slots)).cpu()
        close(got, want, torch.float32, f"steps of {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,blocks", [(48, 3), (40, 5), (256, 1), (320, 4), (24, 24)])
def test_gated_recurrence_in_one_step_and_in_many(dtype, C, blocks):
    """Gates and recurrence against the plain block with an identity convolution and projections."""
    _gated_recurrence_case(dtype, C, blocks, [11, 1, 140], CUTS)


def _short_segments(monkeypatch, ops, rows, lru, wkv):
    """Steps of ``rows`` rows and more are walked in segments of ``lru`` and ``wkv`` rows."""
    monkeypatch.setattr(type(ops), "SCAN_CHUNK_MIN_ROWS", rows)
    monkeypatch.setattr(type(ops), "LRU_SEGMENT", lru)
    monkeypatch.setattr(type(ops), "WKV_SEGMENT", wkv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,blocks,seg", [(48, 3, 8), (320, 4, 5), (130, 1, 16)])
def test_gated_recurrence_walked_in_segments(monkeypatch, dtype, C, blocks, seg):
    """Requests of unequal lengths whose rows are walked in short segments side by side: a request of one segment, one that
    ends on a segment's edge, one that ends just behind an edge; first whole, then the rest in portions that start
    from a state."""
    _short_segments(monkeypatch, ops_of(dtype), 2 * seg, seg, seg)
    lens = [4 * seg, 3, 9 * seg + 1]
    _gated_recurrence_case(dtype, C, blocks, lens, ([1000, 1000, 1000], [3 * seg - 1, 2, 4 * seg + 2], [2 * seg, 1, 2 * seg]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_recurrence_of_a_long_prompt(dtype):
    """A prompt long enough for segments of the usual length, whole and in two portions, beside a short request."""
    _gated_recurrence_case(dtype, 192, 3, [3, 1, 777], ([1000, 1000, 1000], [2, 1, 450]))


def _gated_recurrence_case(dtype, C, blocks, lens, cuts_list):
    ops = ops_of(dtype)
    torch.manual_seed(C + blocks)
    bw = C // blocks
    T = sum(lens)
    u = torch.randn(T, C)
    y = (torch.randn(T, C + 8)).to(dtype)
    t = {"ra": (torch.randn(blocks, bw, bw) * 0.5).to(dtype), "ri": (torch.randn(blocks, bw, bw) * 0.5).to(dtype), "ra.b": torch.randn(blocks, bw),
         "ri.b": torch.randn(blocks, bw), "lam": torch.randn(C) - 2.0, "y.b": torch.randn(C)}
    tp = {k: v.double() for k, v in t.items()}
    want = []
    for s, n in zip([0, lens[0], lens[0] + lens[1]], lens):
        h = u[s:s + n].double()
        want.append(_plain_recurrence(h, y[s:s + n, 8:].double(), tp, C, blocks))
    want = torch.cat(want)
    for cuts in cuts_list:
        state = torch.randn(5, C, device=DEV)  # a slot not yet used holds anything
        state[1:4] = 0.0
        got = torch.zeros(T, C)
        for rows, q0, ql, slots, _ in _steps(lens, cuts):
            a, drive = ops.lru_gates(dev(u[rows]), dev(t["ra"].transpose(1, 2)), dev(t["ri"].transpose(1, 2)), dev(t["ra.b"].reshape(-1)),
                                     dev(t["ri.b"].reshape(-1)), dev(t["lam"]), 8.0)
            got[rows] = ops.lru_scan(a, drive, dev(y[rows]), 8, dev(t["y.b"]), state, i32(q0), i32(ql), i32(slots)).float().cpu()
        close(got, want, dtype, f"steps of {cuts}")


def _plain_recurrence(u, y, t, C, blocks):
    """The recurrence of the plain block on a convolved input ``u`` and a gate branch ``y`` given apart."""
    n = u.shape[0]
    ub = u.view(n, blocks, C // blocks)
    r = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, t["ra"]) + t["ra.b"]).reshape(n, C)
    g = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, t["ri"]) + t["ri.b"]).reshape(n, C)
    a = torch.exp(-8.0 * r * torch.nn.functional.softplus(t["lam"]))
    S, out = torch.zeros(C, dtype=F64), []
    for i in range(n):
        S = a[i] * S + torch.sqrt(1.0 - a[i] ** 2) * (g[i] * u[i])
        out.append(S * P.gelu_tanh(y[i] + t["y.b"]))
    return torch.stack(out)


def test_the_recurrences_gates_agree_with_the_plain_block():
    """The helper above is the plain block's own recurrence: one input, identity projections."""
    C, blocks, n = 12, 3, 9
    torch.manual_seed(1)
    h = torch.randn(n, C, dtype=F64)
    t = {"ra": torch.randn(blocks, 4, 4, dtype=F64), "ri": torch.randn(blocks, 4, 4, dtype=F64), "ra.b": torch.randn(blocks, 4, dtype=F64),
         "ri.b": torch.randn(blocks, 4, dtype=F64), "lam": torch.randn(C, dtype=F64), "y.b": torch.randn(C, dtype=F64), "y": torch.eye(C, dtype=F64),
         "x": torch.eye(C, dtype=F64), "x.b": torch.zeros(C, dtype=F64), "conv": torch.ones(C, 1, dtype=F64), "conv.b": torch.zeros(C, dtype=F64),
         "o": torch.eye(C, dtype=F64)}
    assert torch.allclose(P.rglru(h, t, {"width": C, "blocks": blocks, "conv": 1}), _plain_recurrence(h, h, t, C, blocks))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,width,rank", [(3, 16, 64, 8), (5, 8, 48, 12), (2, 64, 128, 32), (4, 48, 96, 16), (1, 128, 64, 8), (2, 80, 32, 8)])
def test_time_mixing_in_one_step_and_in_many(dtype, H, d, width, rank):
    """Mixes, products, decay and the walk over the tokens, as the mixer strings them together, against the plain mixer."""
    _time_mixing_case(dtype, H, d, width, rank, [11, 1, 90], CUTS)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,width,rank,seg", [(3, 16, 64, 8, 8), (2, 64, 128, 32, 5), (1, 128, 64, 8, 9), (2, 80, 32, 8, 16), (5, 8, 48, 12, 3)])
def test_time_mixing_walked_in_segments(monkeypatch, dtype, H, d, width, rank, seg):
    """As for the gated recurrence: short segments side by side, lengths on, behind and below a segment's edge, portions that
    start from a state."""
    _short_segments(monkeypatch, ops_of(dtype), 2 * seg, seg, seg)
    lens = [4 * seg, 3, 9 * seg + 1]
    _time_mixing_case(dtype, H, d, width, rank, lens, ([1000, 1000, 1000], [3 * seg - 1, 2, 4 * seg + 2], [2 * seg, 1, 2 * seg]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_time_mixing_of_a_long_prompt(dtype):
    """A prompt long enough for segments of the usual length, whole and in two portions, beside a short request."""
    _time_mixing_case(dtype, 3, 64, 96, 16, [3, 1, 600], ([1000, 1000, 1000], [2, 1, 333]))


def _time_mixing_case(dtype, H, d, width, rank, lens, cuts_list):
    ops = ops_of(dtype)
    torch.manual_seed(H * d)
    n = H * d
    T = sum(lens)
    x = torch.randn(T, width)
    t = {f"mu.{m}": torch.rand(width) for m in "rkvgw"}
    t.update({m: (torch.randn(n, width) * width ** -0.5).to(dtype).float() for m in "rkvg"})
    t.update({"w1": (torch.randn(rank, width) * width ** -0.5).to(dtype).float(), "w2": (torch.randn(n, rank) * 0.5).to(dtype).float(),
              "w0": torch.randn(n) * 0.5 - 2.0, "u": torch.randn(H, d) * 0.5, "norm": torch.rand(n) + 0.5, "o": torch.eye(n)})
    tp = {k: v.double() for k, v in t.items()}
    m = {"heads": H, "dim": d}
    want = torch.cat([P.wkv(x[s:s + k].double(), tp, m, 1e-5) for s, k in zip([0, lens[0], lens[0] + lens[1]], lens)])
    mu = torch.stack([t[f"mu.{s}"] for s in "rkvgw"])
    W = {k: dev(t[k], dtype) for k in ("r", "k", "v", "g", "w1", "w2")}
    fill = -rank % 8   # the products sum over multiples of 8: the mixer fills the bottleneck up with zeros, and so does this
    W["w1"], W["w2"] = torch.nn.functional.pad(W["w1"], (0, 0, 0, fill)).contiguous(), torch.nn.functional.pad(W["w2"], (0, fill)).contiguous()
    for cuts in cuts_list:
        prev, state = torch.zeros(5, width, device=DEV), torch.randn(5, H, d, d, device=DEV)  # a slot not yet used holds anything
        state[1:4] = 0.0
        got = torch.zeros(T, n)
        for rows, q0, ql, slots, _ in _steps(lens, cuts):
            seq = (i32(q0), i32(ql), i32(slots))
            mix = ops.shift_mix(dev(x[rows]), prev, dev(mu), *seq)
            r, k, v, g = (ops.linear(mix[i], W[s]) for i, s in enumerate("rkvg"))
            z = ops.linear(ops.tanh_rows(ops.linear(mix[4], W["w1"], None, out_f32=True)), W["w2"], None, out_f32=True)
            got[rows] = ops.wkv(r, k, v, g, z, dev(t["w0"]), dev(t["u"].reshape(-1)), dev(t["norm"]), 1e-5, state, *seq, H, d).float().cpu()
        close(got, want, dtype, f"steps of {cuts}", scale_by=want.abs().max().clamp(min=1.0) * (1 if dtype == torch.float32 else 3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,ff,shared,width", [(6, 2, 24, 40, 64), (3, 3, 8, 8, 48), (7, 1, 24, 0, 48), (32, 4, 32, 64, 128), (5, 3, 12, 0, 40), (70, 64, 8, 0, 64)])
def test_routed_experts_against_the_plain_feed_forward(dtype, E, top, ff, shared, width):
    ops = ops_of(dtype)
    torch.manual_seed(E * ff)
    T = 37
    h = torch.randn(T, width).to(dtype)
    t = {"router": torch.randn(E, width), "router.b": torch.randn(E)}
    for e in range(E):
        t[f"e{e}.up"], t[f"e{e}.down"] = (torch.randn(ff, width) * width ** -0.5).to(dtype).float(), (torch.randn(width, ff) * ff ** -0.5).to(dtype).float()
    mlp = {"router": {"top": top}}
    if shared:
        t["shared.up"], t["shared.down"] = (torch.randn(shared, width) * width ** -0.5).to(dtype).float(), (torch.randn(width, shared) * shared ** -0.5).to(dtype).float()
        mlp["shared"] = {"ff": shared}
    want = P.moe_ff(h.double(), {k: v.double() for k, v in t.items()}, mlp)
    ups, downs = [t[f"e{e}.up"] for e in range(E)], [t[f"e{e}.down"] for e in range(E)]
    if shared:
        ups.append(t["shared.up"]); downs.append(t["shared.down"])
    fill = -(E * ff + shared) % 8
    if fill:
        ups.append(torch.zeros(fill, width)); downs.append(torch.zeros(width, fill))
    gates = ops.route(dev(h), dev(t["router"]), dev(t["router.b"]), top)
    idx, wts = P.route(h.double(), {k: v.double() for k, v in t.items()}, top)
    dense = torch.zeros(T, E, dtype=F64).scatter_(1, idx, wts)
    close(gates, dense, torch.float32, "weights of the chosen experts, zero elsewhere")
    a = ops.expert_act(ops.linear(dev(h), dev(torch.cat(ups), dtype), None, out_f32=True), gates, ff, "gelu")
    got = ops.linear(a, dev(torch.cat(downs, 1), dtype), None, out_f32=True)
    close(got, want, dtype, "the weighted sum of the chosen experts")


def test_a_tie_between_experts_goes_to_the_lower_index():
    ops = ops_of(torch.float32)
    h = torch.zeros(1, 8)
    gates = ops.route(dev(h), dev(torch.randn(5, 8)), dev(torch.tensor([1.0, 3.0, 3.0, 3.0, 0.0])), 2).cpu()
    assert gates[0].tolist() == [0.0, 0.5, 0.5, 0.0, 0.0]


@pytest.mark.parametrize("d", [48, 200, 1030])
def test_norms_behind_the_branches(d):
    ops = ops_of(torch.float32)
    torch.manual_seed(d)
    T, eps = 7, 1e-6
    x, pa, pb = torch.randn(T, d), torch.randn(3, T, d), torch.randn(2, T, d) * 5
    wa, wb, w, bias = torch.rand(d) + 0.5, torch.rand(d) + 0.5, torch.randn(d), torch.randn(d)
    a, b = pa.sum(0).double(), pb.sum(0).double()
    xs = dev(x)
    ops.pair_norm_add(xs, dev(pa), dev(wa), dev(pb), dev(wb), dev(w), eps)
    close(xs, x.double() + P.rms(0.5 * (P.rms(a, eps) * wa.double() + P.rms(b, eps) * wb.double()), eps) * w.double(), torch.float32, "two branches side by side")
    xs = dev(x)
    ops.norm_add_bias(xs, dev(pa), dev(bias), dev(w), eps)
    close(xs, x.double() + P.rms(a + bias.double(), eps) * w.double(), torch.float32, "a branch whose last product has a bias")
    sums = torch.randn(T, 2 * d)
    close(ops.gate_mul(dev(sums), "gelu_tanh"), P.gelu_tanh(sums[:, :d].double()) * sums[:, d:].double(), torch.float32, "gate times up")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,dv,rot,norms", [(4, 2, 16, 24, 8, True), (6, 1, 20, 12, 6, True), (2, 2, 8, 8, 8, False), (8, 2, 48, 96, 48, True),
                                                  (17, 1, 16, 32, 0, True), (4, 4, 64, 64, 32, True)])
def test_rows_of_q_k_and_v_finished(dtype, H, KV, d, dv, rot, norms):
    """Norms over the whole of q and of k, rotation of neighbours, and where keys and values land in their pages."""
    ops = ops_of(dtype)
    torch.manual_seed(H * d + dv)
    T, ps, eps = 21, 16, 1e-6
    dp = -(-max(d, dv) // 16) * 16
    nq, nk, nv = H * d, KV * d, KV * dv
    rows = torch.randn(T, nq + nk + nv + 4)
    qn, kn = (torch.rand(nq) + 0.5, torch.rand(nk) + 0.5) if norms else (None, None)
    pos = torch.arange(3, 3 + T)
    inv = (1000.0 ** (-torch.arange(rot // 2, dtype=F64) * 2 / rot)).float() if rot else None
    slot_map = torch.randperm(3 * ps)[:T].int() + ps
    kp, vp = torch.zeros(5, KV, ps, dp, device=DEV, dtype=dtype), torch.zeros(5, KV, dp, ps, device=DEV, dtype=dtype)
    q = ops.finish_rows(dev(rows), dev(qn), dev(kn), eps, dev(pos.int()), dev(inv), rot, True, dev(slot_map), kp, vp, H, KV, d, dv, ps).float().cpu()
    r = rows.double()
    qw = (P.rms(r[:, :nq], eps) * qn.double() if norms else r[:, :nq]).view(T, H, d)
    kw = (P.rms(r[:, nq:nq + nk], eps) * kn.double() if norms else r[:, nq:nq + nk]).view(T, KV, d)
    if rot:   # the plain rotation counts positions from 0: turn a longer sequence and keep its tail
        lead = lambda x: torch.cat([x.new_zeros(3, *x.shape[1:]), x])
        qw, kw = P.rotate_neighbours(lead(qw), {"base": 1000.0, "dims": rot})[3:], P.rotate_neighbours(lead(kw), {"base": 1000.0, "dims": rot})[3:]
    close(q.view(T, H, dp)[..., :d], qw, dtype, "queries")
    assert float(q.view(T, H, dp)[..., d:].abs().max() if dp > d else 0.0) == 0.0
    page, off = (slot_map // ps).long(), (slot_map % ps).long()
    close(kp.float().cpu()[page, :, off, :d], kw, dtype, "keys in their pages")
    close(vp.float().cpu()[page, :, :dv, off], r[:, nq + nk:nq + nk + nv].view(T, KV, dv), dtype, "values in their pages")


def _attention_case(dtype, H, KV, hd, ps, before, now, seed, chunk, softcap, spike=None, key_splits=0, scale=0.2):
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
    if spike is not None:   # one (request, key) whose score stands out for the first head of each group of the request's last row
        s, key = spike
        page, off = int(table[s, key // ps]), key % ps
        row = sum(now[:s + 1]) - 1
        for kvh in range(KV):
            h = kvh * (H // KV)
            kpool[page, kvh, off] = (q[row, h * hd:(h + 1) * hd] * 4).to(dtype)
        vpool[page, :, :, off] = 50.0
    q = q.to(dtype)
    q0 = torch.tensor([sum(now[:s]) for s in range(S)], dtype=torch.int32)
    ql, p0 = torch.tensor(now, dtype=torch.int32), torch.tensor(before, dtype=torch.int32)
    g = H // KV
    unit = ops.attention_rows_per_block(hd)
    ref.rows_per_block = unit
    work = torch.tensor([[s, r0] for s in range(S) for r0 in range(0, now[s] * g, unit)], dtype=torch.int32)
    want = ref.paged_attention(q, kpool, vpool, table, q0, ql, p0, work, H, KV, hd, ps, None, scale, chunk=chunk, softcap=softcap)
    got = ops.paged_attention(dev(q), dev(kpool), dev(vpool), dev(table), dev(q0), dev(ql), dev(p0), dev(work), H, KV, hd, ps, None, scale,
                              key_splits=key_splits, chunk=chunk, softcap=softcap)
    close(got, want, dtype, f"mixed-batch kernel ({key_splits} splits, chunk {chunk})", scale_by=want.abs().max().clamp(min=1.0))
    if all(n == 1 for n in now) and g <= ops.DECODE_MAX_GROUP:
        got = ops.decode_attention(dev(q), dev(kpool), dev(vpool), dev(table), dev(p0), H, KV, hd, ps, None, scale, chunk=chunk, softcap=softcap)
        close(got, want, dtype, f"decode kernel (chunk {chunk})", scale_by=want.abs().max().clamp(min=1.0))
    return want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk,softcap", [(16, 0.0), (7, 5.0), (64, 50.0), (100, 0.0), (0, 2.0), (1, 0.0)])
@pytest.mark.parametrize("H,KV,hd", [(8, 2, 96), (6, 1, 32), (4, 4, 80), (17, 1, 32)])
def test_attention_over_chunks_with_capped_scores(dtype, chunk, softcap, H, KV, hd):
    _attention_case(dtype, H, KV, hd, 16, [0, 5, 130], [150, 1, 9], 1, chunk, softcap)
    _attention_case(dtype, H, KV, hd, 16, [0, 5, 130], [40, 1, 9], 2, chunk, softcap, key_splits=3)
    _attention_case(dtype, H, KV, hd, 16, [600, 17, 0, 255], [1, 1, 1, 1], 3, chunk, softcap)
    _attention_case(dtype, H, KV, hd, 64, [1000], [1], 4, chunk, softcap)


def test_a_cap_far_below_the_scores_flattens_the_softmax():
    """Scores of +-40 under a cap of 0.01 weigh every key alike: the output is the mean of the values."""
    ops = ops_of(torch.float32)
    hd, ps, n = 16, 16, 11
    torch.manual_seed(2)
    kpool, vpool = torch.randn(2, 1, ps, hd) * 10, torch.randn(2, 1, hd, ps)
    q = torch.randn(1, hd) * 10
    got = ops.decode_attention(dev(q), dev(kpool), dev(vpool), i32([[1]]), i32([n - 1]), 1, 1, hd, ps, None, 1.0, chunk=0, softcap=0.01).cpu()
    assert float((got[0] - vpool[1, 0, :, :n].mean(-1)).abs().max()) < 2e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("chunk,n,key,seen", [(64, 800, 768, True), (64, 800, 767, False), (64, 800, 799, True), (64, 769, 768, True), (64, 769, 767, False),
                                              (64, 768, 704, True), (64, 768, 703, False), (100, 800, 700, True), (100, 800, 699, False), (100, 800, 0, False),
                                              (1000, 800, 0, True), (1000, 800, 15, True), (1000, 800, 16, True), (24, 50, 47, False), (24, 50, 48, True),
                                              (0, 800, 0, True), (0, 800, 400, True)])
def test_a_key_that_stands_out_is_seen_only_inside_the_rows_chunk(dtype, decoded, chunk, n, key, seen):
    """The last row of ``n`` and one key whose score stands out: the first key of the row's chunk and the last of the chunk
    before it, the first key of all under a chunk longer than the sequence, keys at page borders, the row itself.  Where
    the key is seen its value (50 in every column) comes out; where not, values of order one."""
    want = _attention_case(dtype, 6, 1, 80, 16, [n - 1] if decoded else [0], [1] if decoded else [n], 5, chunk, 30.0, spike=(0, key), scale=0.5)
    top = float(want[-1, :80].min())
    assert top > 25.0 if seen else top < 10.0


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
    d = U.make_dir(tmp_path, name, seed=10, sharpen=sharpen_for(dtype))
    toks = U.tokens_of(330, U.CONFIGS[name]["vocab"], 3)
    lm = loaded(d, dtype, max_tokens=512)
    got = U.run_schedule(lm, {"a": toks}, [[("a", 10)]] + [[("a", 1)]] * 320)["a"]
    assert U.within(got, plain_for(d, dtype, toks), dtype)
    assert len(lm.step._graphs) > 0     # the single rows ran from captured steps


def test_a_long_prompt_in_portions_behind_pages_of_64(tmp_path):
    """Recurrences over a thousand tokens and chunks across many pages, in a step of many rows and in portions that end
    inside pages and chunks."""
    d = U.make_dir(tmp_path, "mixed", seed=11)
    toks = U.tokens_of(1100, 97, 6)
    want = plain_for(d, torch.float32, toks)
    lm = loaded(d, torch.float32, page_size=64, max_tokens=1152)
    for what, schedule in {"whole": [[("a", 1100)]], "portions": _cut("a", 1100, [500, 63, 2, 129, 300, 7])}.items():
        got = U.run_schedule(lm, {"a": toks}, schedule)["a"]
        assert U.relative_error(got, want) < F32, what


def test_long_portions_beside_decoded_tokens(tmp_path):
    """Steps whose rows are many enough for the recurrences' segments while some requests bring one row: two long
    portions side by side, then a long portion beside two requests that decode."""
    d = U.make_dir(tmp_path, "mixed", seed=21)
    reqs = {"a": U.tokens_of(700, 97, 1), "b": U.tokens_of(420, 97, 2), "c": U.tokens_of(9, 97, 3)}
    schedule = [[("a", 290), ("b", 300)], [("c", 7), ("b", 118)], [("b", 1), ("a", 405), ("c", 1)], [("b", 1), ("a", 5), ("c", 1)]]
    lm = loaded(d, torch.float32, page_size=64, max_tokens=1344, max_requests=3)
    got = U.run_schedule(lm, reqs, schedule)
    for i, toks in reqs.items():
        assert U.relative_error(got[i], plain_for(d, torch.float32, toks)) < F32, i


def test_sizes_the_recurrences_do_not_take_are_refused_when_the_part_is_built():
    """Blocks of the recurrence wider than the gates' kernel holds, and heads of time mixing beyond its registers, are
    refused with the size when the part is built, not at the first step."""
    from machserve_amd.config import GatedRecurrenceSpec, TimeMixSpec
    from machserve_amd.parts import MIXERS, Runtime
    rt = Runtime(torch.device(DEV), torch.bfloat16, ops_of(torch.bfloat16))
    most = rt.ops.linrec_limits()["lru_block"]
    MIXERS.build(GatedRecurrenceSpec("gated_recurrence", 64, 2 * most, 2, 4), rt)
    with pytest.raises(ValueError, match=f"blocks of {2 * most}"):
        MIXERS.build(GatedRecurrenceSpec("gated_recurrence", 64, 2 * most, 1, 4), rt)
    with pytest.raises(ValueError, match="heads of 136"):
        MIXERS.build(TimeMixSpec("time_mix", 64, 2, 136, 8, 1e-5), rt)


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


def test_a_state_lost_would_show(tmp_path):
    """The test's own power: the same request with its slot's states zeroed half way is far from the plain model."""
    d = U.make_dir(tmp_path, "mixed", seed=16)
    toks = U.tokens_of(60, 97, 9)
    want = plain_for(d, torch.float32, toks)
    lm = loaded(d, torch.float32, use_graphs=False)
    from machserve_amd.engine.step import StepEntry
    slot = lm.cache.admit()
    lm.step([StepEntry(slot, toks[:30], [])])
    lm.device_cache.zero_state(slot)
    got = lm.step([StepEntry(slot, toks[30:], list(range(30)))]).float().cpu()
    lm.cache.release(slot)
    assert U.relative_error(got, want[30:]) > 1e-2


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
