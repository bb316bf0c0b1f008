"""Small Melerax configurations, model folders made from them and the plain model's logits."""
from __future__ import annotations

import json
import os

import torch

from plain import melerax_plain as P
from renanex_util import relative_error, relative_errors, run_schedule, tokens_of, within  # noqa: F401  (shared runners)


def attention(heads, kv, dim, vdim, scale, conv=4, rot=(10000.0, None), softcap=30.0, chunk=16):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1] or dim}
    if softcap:
        m["softcap"] = softcap
    if chunk:
        m["mask"] = {"size": chunk}
    return m


def recurrence(width, blocks, conv):
    return {"width": width, "blocks": blocks, "conv": conv}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(width, vocab, layers, eps=1e-6, bigram=(53, 7, 3)):
    return {"architecture": "Melerax", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}, "layers": layers}


CONFIGS = {
    # every kind of layer and of feed-forward once or twice; values wider than keys; a rotation of part of a head
    "mixed": model(64, 97, [
        layer("parallel", {"left": attention(4, 2, 16, 24, 0.4, conv=3, rot=(500.0, 8), chunk=16), "right": recurrence(48, 3, 2)}, dense(80)),
        layer("wkv", {"heads": 3, "dim": 16, "rank": 8}, moe(6, 2, 24, shared=40)),
        layer("rglru", recurrence(80, 2, 4), dense(72)),
        layer("parallel", {"left": attention(4, 4, 16, 16, 0.35, conv=2, chunk=24), "right": recurrence(32, 1, 3)}, moe(5, 3, 16)),
        layer("wkv", {"heads": 2, "dim": 32, "rank": 16}, None)]),
    # sizes that are no multiples of 16, chunks that are no multiples of a page or a tile, one key/value head under six
    # heads, values narrower than keys, one expert a token, every expert a token, a bottleneck that is no multiple of 8,
    # one tap (no state) and five, a layer without feed-forward, heads x size beside the width
    "odd": model(48, 61, [
        layer("rglru", recurrence(40, 5, 1), moe(3, 3, 8, shared=8)),
        layer("parallel", {"left": attention(6, 1, 20, 12, 0.3, conv=5, rot=(100.0, 6), softcap=5.0, chunk=7), "right": recurrence(24, 4, 5)}, None),
        layer("wkv", {"heads": 5, "dim": 8, "rank": 12}, moe(7, 1, 24)),
        layer("parallel", {"left": attention(2, 2, 8, 8, 0.7, conv=1, rot=(10000.0, 8), softcap=100.0, chunk=33), "right": recurrence(16, 2, 2)}, dense(40))],
        eps=1e-5, bigram=(11, 1, 1)),
    # heads of 64 numbers (the attention kernels' tile of 64 takes work items of another size in the two-byte types), a
    # chunk longer than the prompts of most tests, seventeen heads over one key/value head (beyond a decode tile), wide
    # recurrence blocks, many experts
    "wide": model(128, 128, [
        layer("parallel", {"left": attention(4, 4, 64, 64, 0.15, conv=4, rot=(250000.0, 32), chunk=200), "right": recurrence(256, 2, 3)}, moe(32, 4, 32, shared=64)),
        layer("wkv", {"heads": 2, "dim": 64, "rank": 32}, dense(256)),
        layer("parallel", {"left": attention(17, 1, 16, 32, 0.3, conv=2, rot=(1000.0, 16), chunk=32), "right": recurrence(64, 8, 4)}, dense(96))],
        bigram=(257, 31, 5)),
}


def make_dir(tmp, name: str, seed: int = 0, sharpen: float = 6.0, dtype=torch.float32) -> str:
    """A model folder of random weights, changed so that faults show: embeddings and the mixers' input projections of order
    one (the gates and decays then depend on the token), query norms times ``sharpen`` (softmaxes far from flat: a key
    that is missing or one too many shows in the logits), slow decays in both recurrences (a state that is lost or kept
    from another request shows many tokens later)."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights import write_random_model
    out = os.path.join(str(tmp), f"melerax_{name}_{seed}")
    write_random_model(dict(CONFIGS[name]), seed, out, dtype)
    path = os.path.join(out, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        t = w[k].float()
        if k in ("embed", "bigram"):
            t = t * 40.0
        elif k.endswith(".q.norm"):
            t = t * sharpen
        elif k.endswith((".x", ".y", ".mix.r", ".mix.k", ".mix.v", ".mix.g", ".mix.w1", ".left.q", ".left.k", ".left.v", ".up", ".gate")):
            t = t * 8.0
        elif k.endswith(".lam"):
            t = t - 2.5
        elif k.endswith(".w0"):
            t = t - 2.0
        elif k.endswith((".ls1", ".ls2")):
            t = t * 0.7
        w[k] = t.to(dtype)
    save_file(w, path)
    return out


def read(model_dir: str):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return load_file(os.path.join(model_dir, "model.safetensors")), cfg


def plain_logits(model_dir: str, tokens, dtype=torch.float64, weights_as=None) -> torch.Tensor:
    """The plain model's logits; ``weights_as``: matrices rounded to this type first, as a run in that type holds them."""
    w, cfg = read(model_dir)
    if weights_as is not None and weights_as != torch.float32:
        w = {k: v.to(weights_as).float() if _is_matrix(k, v) else v for k, v in w.items()}
    return P.forward(w, cfg, tokens, dtype)


def _is_matrix(name: str, t) -> bool:
    """What a run keeps in its element type: operands of matrix products and the two tables (not filters, not the router)."""
    if name.endswith((".conv", ".router", ".u")) or t.dim() < 2:
        return False
    return True
