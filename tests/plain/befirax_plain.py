"""Plain, slow Befirax decoder: whole sequences, no cache, one function per mechanism.

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


def rms_norm(x, w, eps):
    return rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ pieces shared by the mixers
def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``u [n, channels]``, ``w [channels, taps]``: the last column of ``w`` meets the current token, the one before it
    the token before, and so on; what lies before the sequence is zero."""
    n, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(n):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def angles(n: int, base: float, dims: int, dtype, pos0: int = 0) -> torch.Tensor:
    """``[n, dims / 2]``: position times ``base^(-2i / dims)``."""
    i = torch.arange(dims // 2, dtype=dtype)
    freq = torch.pow(torch.tensor(float(base), dtype=dtype), -2.0 * i / dims)
    return torch.arange(pos0, pos0 + n, dtype=dtype)[:, None] * freq[None, :]


def rotate_neighbours(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """``x [n, heads, d]``: the first ``dims`` numbers of every head turned in pairs ``(2i, 2i + 1)``."""
    a = angles(x.shape[0], base, dims, x.dtype)[:, None, :]
    c, s = torch.cos(a), torch.sin(a)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def rotate_halves(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """``x [n, heads, d]``: the first ``dims`` numbers of every head turned in pairs ``(i, i + dims / 2)``."""
    a = angles(x.shape[0], base, dims, x.dtype)[:, None, :]
    c, s = torch.cos(a), torch.sin(a)
    half = dims // 2
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(n: int, window=None) -> torch.Tensor:
    """``[n, n]`` booleans: row i sees column j if ``j <= i`` and, under a window, ``i - j < window``."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    return ok


def softmax_rows(scores: torch.Tensor, ok: torch.Tensor) -> torch.Tensor:
    return torch.softmax(scores.masked_fill(~ok, float("-inf")), dim=-1)


# ------------------------------------------------------------------ differential attention
def diff_lambda(t, p: str, diff: float, dtype) -> torch.Tensor:
    g = lambda name: t[p + name].to(dtype)
    return torch.exp((g("lq1") * g("lk1")).sum()) - torch.exp((g("lq2") * g("lk2")).sum()) + diff


def diff_keys_values(t, p: str, m: dict, h: torch.Tensor):
    """Keys ``[n, G, 2, dim]`` (convolved, rotated) and values ``[n, G, vdim]`` (convolved) of a layer that has them."""
    dt = h.dtype
    n, G, d, dv = h.shape[0], int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = h @ t[p + "k"].to(dt).T + t[p + "k.b"].to(dt)
    v = h @ t[p + "v"].to(dt).T + t[p + "v.b"].to(dt)
    if m.get("conv"):
        k, v = causal_conv(k, t[p + "k.conv"].to(dt)), causal_conv(v, t[p + "v.conv"].to(dt))
    k = k.view(n, G * 2, d)
    if m.get("rot"):
        k = rotate_neighbours(k, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    return k.view(n, G, 2, d), v.view(n, G, dv)


def diff_attention(t, p: str, m: dict, h: torch.Tensor, eps: float, kv=None):
    """Two softmax maps per head over the same values, the second subtracted ``lambda`` times; the head's result
    divided by its root mean square and multiplied by ``1 - diff``; a sigmoid gate; the output projection.  ``kv``: the
    keys and values of another layer to use instead of this one's own.  Returns ``(output [n, w], (keys, values))``."""
    dt = h.dtype
    n, H, G, d, dv = h.shape[0], int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    q = h @ t[p + "q"].to(dt).T + t[p + "q.b"].to(dt)
    if m.get("conv"):
        q = causal_conv(q, t[p + "q.conv"].to(dt))
    q = q.view(n, H * 2, d)
    if m.get("rot"):
        q = rotate_neighbours(q, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    q = q.view(n, H, 2, d)
    if kv is None:
        kv = diff_keys_values(t, p, m, h)
    k, v = kv
    lam = diff_lambda(t, p, diff, dt)
    ok = visible(n)
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = [softmax_rows((q[:, a, j] @ k[:, g, j].T) * float(m["scale"]), ok) @ v[:, g] for j in (0, 1)]
        o = maps[0] - lam * maps[1]
        heads.append(rms(o, eps) * (1.0 - diff))
    o = torch.cat(heads, dim=-1) * torch.sigmoid(h @ t[p + "g"].to(dt).T)
    return o @ t[p + "o"].to(dt).T + t[p + "o.b"].to(dt), kv


# ------------------------------------------------------------------ attention through a latent
def latent_attention(t, p: str, m: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """Per token one normed latent and one rotated key part for all heads; a head's key is ``[W_uk c | rotated part]``,
    its value ``W_uv c``; a window of ``mask.size`` positions; a sigmoid gate per head."""
    dt = h.dtype
    n, H, d, r, dv, rank = h.shape[0], int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    base = float(m["rot"]["base"])
    q = (h @ t[p + "q"].to(dt).T).view(n, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_halves(q[..., d:], base, r)
    down = h @ t[p + "dkv"].to(dt).T
    c = rms_norm(down[:, :rank], t[p + "dkv.norm"].to(dt), eps)
    k_rot = rotate_halves(down[:, rank:].reshape(n, 1, r), base, r)[:, 0]
    k_plain = (c @ t[p + "uk"].to(dt).T).view(n, H, d)
    v = (c @ t[p + "uv"].to(dt).T).view(n, H, dv)
    window = int(m["mask"]["size"]) if m.get("mask") else None
    ok = visible(n, window)
    gate = torch.sigmoid(h @ t[p + "g"].to(dt).T)  # [n, H]
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * float(m["scale"])
        heads.append((softmax_rows(s, ok) @ v[:, a]) * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ t[p + "o"].to(dt).T


# ------------------------------------------------------------------ state-space layer
def mamba2(t, p: str, m: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """``S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T``, ``y_t = S_t^T C_t + D x_t`` per head, behind a convolution
    with SiLU on x, B and C; ``y silu(z)`` normed in groups; the output projection."""
    dt_ = h.dtype
    n, H, P, N, G = h.shape[0], int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * P
    u = h @ t[p + "in"].to(dt_).T
    z, xbc, step = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t[p + "conv"].to(dt_)) + t[p + "conv.b"].to(dt_))
    x = xbc[:, :inner].reshape(n, H, P)
    B = xbc[:, inner:inner + G * N].reshape(n, G, N)
    C = xbc[:, inner + G * N:].reshape(n, G, N)
    step = softplus(step + t[p + "dt_bias"].to(dt_))  # [n, H]
    rate = torch.exp(t[p + "A_log"].to(dt_))  # [H]
    skip = t[p + "D"].to(dt_)
    S = torch.zeros((H, N, P), dtype=dt_)
    y = torch.zeros((n, H, P), dtype=dt_)
    for i in range(n):
        for a in range(H):
            g = a // (H // G)
            S[a] = torch.exp(-rate[a] * step[i, a]) * S[a] + step[i, a] * torch.outer(B[i, g], x[i, a])
            y[i, a] = S[a].T @ C[i, g] + skip[a] * x[i, a]
    y = y.reshape(n, inner) * silu(z)
    parts = int(m["norm_groups"])
    y = rms(y.view(n, parts, inner // parts), eps).reshape(n, inner) * t[p + "norm"].to(dt_)
    return y @ t[p + "o"].to(dt_).T


# ------------------------------------------------------------------ feed-forward of routed experts
def route(t, p: str, mlp: dict, h: torch.Tensor):
    """``(chosen [n, top], weights [n, top])``: softmax over all router outputs; the choice adds a correction to the
    scores, the weights are the chosen scores themselves over their sum."""
    z = h @ t[p + "router"].to(h.dtype).T
    s = torch.softmax(z, dim=-1)
    pick = s + t[p + "correction"].to(h.dtype)
    chosen = torch.topk(pick, int(mlp["router"]["top"]), dim=-1).indices
    w = torch.gather(s, 1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + 1e-20)


def expert(t, p: str, e: int, h: torch.Tensor) -> torch.Tensor:
    dt = h.dtype
    return (silu(h @ t[p + f"e{e}.gate"].to(dt).T) * (h @ t[p + f"e{e}.up"].to(dt).T)) @ t[p + f"e{e}.down"].to(dt).T


def moe(t, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    """Every row's chosen experts, each run by itself; the router's last ``identity`` outputs stand for experts that
    return their input."""
    real = int(mlp["router"]["experts"])
    chosen, w = route(t, p, mlp, h)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, g in zip(chosen[i].tolist(), w[i]):
            out[i] += g * (expert(t, p, e, h[i:i + 1])[0] if e < real else h[i])
    return out


# ------------------------------------------------------------------ several residual streams
def streams_read(t, p: str, xs: torch.Tensor) -> torch.Tensor:
    """``xs [s, n, w]``: the sublayer's input, the streams weighted by ``in``."""
    return torch.einsum("s,snw->nw", t[p + "in"].to(xs.dtype), xs)


def streams_write(t, p: str, xs: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """New streams from the old ones: ``x_t = sum_s mix[s, t] x_s + out[t] y``."""
    return torch.einsum("st,snw->tnw", t[p + "mix"].to(xs.dtype), xs) + t[p + "out"].to(xs.dtype)[:, None, None] * y[None]


# ------------------------------------------------------------------ the model
def forward(t, cfg: dict, tokens, dtype=torch.float64, layers_out=None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of one sequence.  ``layers_out``: a list that receives the sum of the streams after every layer."""
    eps = float(cfg["norm"]["eps"])
    hyper = cfg.get("streams") is not None  # several streams with learned reads and writes; else the plain residual sum
    s = int(cfg["streams"]) if hyper else 1
    x = t["embed"].to(dtype)[torch.as_tensor(list(tokens), dtype=torch.long)]
    xs = x[None].repeat(s, 1, 1)
    caches = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]

        def mixer(h):
            if layer["type"] == "attention":
                src = m.get("kv_from")
                y, kv = diff_attention(t, p, m, h, eps, None if src is None else caches[int(src)])
                caches[i] = kv
                return y
            if layer["type"] == "latent_attention":
                return latent_attention(t, p, m, h, eps)
            if layer["type"] == "mamba2":
                return mamba2(t, p, m, h, eps)
            raise ValueError(layer["type"])

        subs = [(mixer, "norm1", "hc1.")]
        if layer.get("mlp") is not None:
            subs.append((lambda h: moe(t, f"l{i}.mlp.", layer["mlp"], h), "norm2", "hc2."))
        for fn, norm, hc in subs:
            if hyper:
                y = fn(rms_norm(streams_read(t, f"l{i}.{hc}", xs), t[f"l{i}.{norm}"].to(dtype), eps))
                xs = streams_write(t, f"l{i}.{hc}", xs, y)
            else:
                xs = xs + fn(rms_norm(xs[0], t[f"l{i}.{norm}"].to(dtype), eps))[None]
        if layers_out is not None:
            layers_out.append(xs.sum(0))
    x = rms_norm(xs.sum(0), t["final.norm"].to(dtype), eps)
    return x @ t["embed"].to(dtype).T


def greedy_generate(t, cfg: dict, prompt, new_tokens: int, dtype=torch.float64):
    seq = list(prompt)
    for _ in range(new_tokens):
        seq.append(int(forward(t, cfg, seq, dtype)[-1].argmax()))
    return seq[len(prompt):]
