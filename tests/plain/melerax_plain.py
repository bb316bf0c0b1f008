"""Plain, slow Melerax decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Input is a dict of tensors by checkpoint name and the
config.json dict; everything is computed with ordinary torch operations on the CPU in
``dtype`` (float32 or float64), token after token where the design is a recurrence.

Notation: ``n`` tokens, width ``w``; a linear map is ``y = x @ W.T`` with ``W [out, in]``.
"""
from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Rows divided by ``sqrt(mean(x^2) + eps)``."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ embedding
def bigram_rows(tokens, mul_prev: int, mul_cur: int, buckets: int):
    """Row of the bigram table for every token: a hash of the pair (previous, current); the last row for the first token."""
    rows = [buckets]
    for p, c in zip(tokens[:-1], tokens[1:]):
        rows.append((int(p) * mul_prev + int(c) * mul_cur) % buckets)
    return torch.tensor(rows, dtype=torch.long)


def embed(tensors, cfg, tokens, dtype):
    x = tensors["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + tensors["bigram"].to(dtype)[bigram_rows(list(tokens), int(bg["mul_prev"]), int(bg["mul_cur"]), int(bg["buckets"]))]
    return x


# ------------------------------------------------------------------ pieces of the mixers
def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``u [n, channels]``, ``w [channels, taps]``: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start."""
    n, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * u[s]
    return y


def rotate_neighbours(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [n, heads, d]``: of the first ``dims`` numbers of a head, neighbours ``(2i, 2i + 1)`` at position p turn by
    ``p * base^(-2i / dims)``; the rest pass."""
    dims, base = int(rot["dims"]), float(rot["base"])
    n = x.shape[0]
    out = x.clone()
    for p in range(n):
        for i in range(dims // 2):
            a = p * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[p, :, 2 * i], x[p, :, 2 * i + 1]
            out[p, :, 2 * i] = u * c - v * s
            out[p, :, 2 * i + 1] = v * c + u * s
    return out


def chunk_visible(n: int, size: int) -> torch.Tensor:
    """``[n, n]`` bool: row i sees j <= i of its own chunk of ``size`` positions, chunks counted from position 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i // size) == (j // size))


# ------------------------------------------------------------------ mixers
def chunked_attention(h, t, m, eps):
    """Grouped-query attention behind a short convolution on q, k and v, with norms over the whole q and k projections,
    a rotation of neighbours, capped scores and a mask of chunks."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ t["q"].T + t["q.b"]
    k = h @ t["k"].T + t["k.b"]
    v = h @ t["v"].T + t["v.b"]
    if m.get("conv"):
        q, k, v = causal_conv(q, t["q.conv"]), causal_conv(k, t["k.conv"]), causal_conv(v, t["v.conv"])
    q = rms(q, eps) * t["q.norm"]
    k = rms(k, eps) * t["k.norm"]
    q, k, v = q.view(n, H, d), k.view(n, G, d), v.view(n, G, dv)
    if m.get("rot"):
        q, k = rotate_neighbours(q, m["rot"]), rotate_neighbours(k, m["rot"])
    k_of = torch.arange(H) // (H // G)
    s = torch.einsum("ihd,jhd->hij", q, k[:, k_of]) * float(m["scale"])
    cap = m.get("softcap")
    if cap:
        s = float(cap) * torch.tanh(s / float(cap))
    mask = m.get("mask")
    see = chunk_visible(n, int(mask["size"])) if mask else torch.ones(n, n, dtype=torch.bool).tril()
    p = torch.softmax(s.masked_fill(~see, float("-inf")), -1)
    o = torch.einsum("hij,jhd->ihd", p, v[:, k_of])
    return o.reshape(n, -1) @ t["o"].T


def rglru(h, t, m):
    """Recurrent block: a gelu branch y, a convolved branch u, gates from u block by block, and the recurrence
    ``S <- a S + sqrt(1 - a^2) (i * u)`` with ``a = exp(-8 r softplus(lam))``; the output is ``W_o (S * y)``."""
    n = h.shape[0]
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(h @ t["y"].T + t["y.b"])
    u = causal_conv(h @ t["x"].T + t["x.b"], t["conv"]) + t["conv.b"]
    ub = u.view(n, blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, t["ra"]) + t["ra.b"]).reshape(n, width)
    g = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, t["ri"]) + t["ri.b"]).reshape(n, width)
    log_a = -8.0 * r * torch.nn.functional.softplus(t["lam"])
    a = torch.exp(log_a)
    S = torch.zeros(width, dtype=h.dtype)
    out = []
    for i in range(n):
        S = a[i] * S + torch.sqrt(1.0 - a[i] ** 2) * (g[i] * u[i])
        out.append(S * y[i])
    return torch.stack(out) @ t["o"].T


def wkv(h, t, m, eps):
    """Time mixing with a decay per key channel that depends on the token, and a bonus for the current token."""
    n, w = h.shape
    H, d = m["heads"], m["dim"]
    prev = torch.cat([h.new_zeros(1, w), h[:-1]], 0)

    def mix(name):
        return h + (prev - h) * t["mu." + name]
    r = (mix("r") @ t["r"].T).view(n, H, d)
    k = (mix("k") @ t["k"].T).view(n, H, d)
    v = (mix("v") @ t["v"].T).view(n, H, d)
    gate = silu(mix("g") @ t["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ t["w1"].T) @ t["w2"].T + t["w0"])).view(n, H, d)
    u = t["u"]
    S = h.new_zeros(H, d, d)   # [head, key channel, value channel]
    out = []
    for i in range(n):
        kv = k[i][:, :, None] * v[i][:, None, :]
        out.append(torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[i]))
        S = decay[i][:, :, None] * S + kv
    o = rms(torch.stack(out), eps).reshape(n, H * d)
    return (o * t["norm"] * gate) @ t["o"].T


def parallel(h, t, m, eps):
    """Two mixers side by side: each output RMS-normed with its own weight, half their sum."""
    left = chunked_attention(h, _strip(t, "left."), m["left"], eps)
    right = rglru(h, _strip(t, "right."), m["right"])
    return 0.5 * (rms(left, eps) * t["left.out"] + rms(right, eps) * t["right.out"])


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, t):
    return (gelu_tanh(h @ t["gate"].T + t["gate.b"]) * (h @ t["up"].T + t["up.b"])) @ t["down"].T + t["down.b"]


def route(h, t, top: int):
    """``(experts [n, top], weights [n, top])``: the largest logits, softmax over the chosen ones only."""
    z = h @ t["router"].T + t["router.b"]
    best, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(best, -1)


def expert(h, up, down):
    return gelu_erf(h @ up.T) @ down.T


def moe_ff(h, t, mlp):
    idx, wts = route(h, t, int(mlp["router"]["top"]))
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, g in zip(idx[i].tolist(), wts[i]):
            out[i] = out[i] + g * expert(h[i], t[f"e{e}.up"], t[f"e{e}.down"])
    if mlp.get("shared"):
        out = out + expert(h, t["shared.up"], t["shared.down"])
    return out


# ------------------------------------------------------------------ the model
def _strip(t, prefix):
    return {k[len(prefix):]: v for k, v in t.items() if k.startswith(prefix)}


def _sub(tensors, prefix, dtype):
    return {k[len(prefix):]: v.to(dtype) for k, v in tensors.items() if k.startswith(prefix)}


def mixer_of(layer, h, t, eps):
    kind, m = layer["type"], layer["mixer"]
    if kind == "parallel":
        return parallel(h, t, m, eps)
    if kind == "rglru":
        return rglru(h, t, m)
    if kind == "wkv":
        return wkv(h, t, m, eps)
    raise ValueError(f"unknown layer type {kind!r}")


def forward(tensors, cfg, tokens, dtype=torch.float64, streams=None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of one sequence.  ``streams``: a list that receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tensors, cfg, tokens, dtype)
    for i, layer in enumerate(cfg["layers"]):
        g = lambda name: tensors[f"l{i}.{name}"].to(dtype)
        y = mixer_of(layer, x, _sub(tensors, f"l{i}.mix.", dtype), eps)
        x = x + norm_one_plus(y, g("norm1"), eps) * g("ls1")
        mlp = layer.get("mlp")
        if mlp is not None:
            t = _sub(tensors, f"l{i}.mlp.", dtype)
            y = dense_ff(x, t) if mlp["kind"] == "dense" else moe_ff(x, t, mlp)
            x = x + norm_one_plus(y, g("norm2"), eps) * g("ls2")
        if streams is not None:
            streams.append(x.clone())
    x = norm_one_plus(x, tensors["final.norm"].to(dtype), eps)
    return x @ tensors["head"].to(dtype).T


def greedy_generate(tensors, cfg, prompt, n_new: int, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(tensors, cfg, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]
