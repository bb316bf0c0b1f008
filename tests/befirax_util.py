"""Small Befirax configurations, model folders made from them and the plain model's logits."""
from __future__ import annotations

import json
import os

import torch

from plain import befirax_plain as P
from renanex_util import relative_error, relative_errors, run_schedule, tokens_of  # noqa: F401  (shared runners)


def attention(heads, kv, dim, vdim, scale, diff, conv=3, rot=(10000.0, None), kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if conv:
        m["conv"] = conv
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1] or dim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": {"base": base, "dims": rot_dim}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def mamba2(heads, vdim, state, groups, conv, parts):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": parts}}


def moe(experts, top, ff, identity=0):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def model(width, vocab, layers, eps=1e-6, streams=None):
    out = {"architecture": "Befirax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    return out


CONFIGS = {
    # three streams; every mixer twice, with other sizes the second time; a layer that reads another's keys and values; a
    # window that is no multiple of a page; a layer without feed-forward; values wider than keys
    "mixed": model(64, 97, [
        layer(attention(4, 2, 16, 24, 0.3, 0.25, conv=3, rot=(500.0, 8)), moe(6, 2, 24, identity=1)),
        layer(mamba2(4, 16, 8, 2, 3, 2), moe(5, 3, 16, identity=2)),
        layer(latent(3, 16, 8, 16, 24, 0.2, base=1000.0, window=20), None),
        layer(attention(4, 2, 16, 24, 0.25, 0.4, conv=2, rot=(500.0, 8), kv_from=0), moe(6, 2, 24, identity=1)),
        layer(mamba2(2, 32, 16, 1, 4, 1), moe(4, 1, 8, identity=1)),
        layer(latent(2, 8, 16, 24, 40, 0.25, base=50.0), moe(3, 2, 16))], streams=3),
    # one residual stream with the plain sum; sizes that are no multiples of 8 or 16; one key/value head under six heads;
    # values narrower than keys; one tap (no state) and no rotation; every expert a token; one expert a token; groups
    # as many as heads; a window shorter than a page; an attention layer first and last
    "odd": model(48, 61, [
        layer(attention(6, 1, 20, 10, 0.3, 0.1, conv=1, rot=None), moe(3, 3, 8)),
        layer(mamba2(3, 8, 5, 3, 2, 3), moe(7, 1, 24, identity=3)),
        layer(latent(5, 8, 6, 12, 20, 0.3, base=100.0, window=7), moe(2, 2, 8, identity=2)),
        layer(attention(2, 2, 8, 8, 0.5, 0.6, conv=5, rot=(10000.0, 8)), None)], eps=1e-5),
    # one stream that is read and written with weights; heads of 64 (the attention kernels' tile of 64 takes work items
    # of another size in the two-byte types); seventeen heads over one latent (beyond a decode tile); many states; a
    # window longer than most tests' prompts; many experts
    "wide": model(128, 128, [
        layer(mamba2(2, 64, 64, 1, 4, 1), moe(32, 4, 32, identity=4)),
        layer(attention(2, 2, 64, 64, 0.15, 0.3, conv=4, rot=(250000.0, 32)), moe(4, 2, 64)),
        layer(latent(17, 16, 16, 32, 48, 0.3, base=1000.0, window=200), moe(8, 8, 16, identity=1))], streams=1),
}

# configurations for the GPU alone (the stand-ins would take minutes): sizes nearer a real model's layers
MORE_CONFIGS = {
    # four streams; an attention layer first; heads of 64 with values of 128; a latent of 128 beside a rotated part of 64
    # and one of 160 beside 32; state-space heads of 64 and 128 with 64 and 128 states; sixteen experts; a layer without
    # feed-forward in the middle; the reading layer convolves with other taps than the layer it reads
    "big": model(512, 1000, [
        layer(attention(8, 2, 64, 128, 0.125, 0.2, conv=2, rot=(10000.0, 64)), moe(16, 4, 128, identity=3)),
        layer(latent(8, 64, 64, 64, 128, 0.09, base=250000.0, window=64), moe(8, 2, 256)),
        layer(mamba2(16, 64, 64, 4, 4, 4), moe(16, 4, 128, identity=3)),
        layer(attention(8, 2, 64, 128, 0.125, 0.35, conv=4, rot=(10000.0, 64), kv_from=0), moe(8, 2, 256)),
        layer(mamba2(8, 128, 128, 1, 2, 1), None),
        layer(latent(4, 128, 32, 128, 160, 0.08, base=10000.0), moe(16, 1, 64, identity=1))], streams=4),
}
CONFIGS_ALL = dict(CONFIGS, **MORE_CONFIGS)


def make_dir(tmp, name: str, seed: int = 0, sharpen: float = 6.0, dtype=torch.float32, experts: float = 8.0) -> str:
    """A model folder of random weights, changed so that faults show: embeddings of order one, query and key projections
    times ``sharpen`` (softmaxes far from flat: a key that is missing or one too many shows in the logits), input
    projections of the state-space layers and of the experts of order one, corrections large enough to change the
    choice, streams that differ from each other.  ``experts``: the factor on the experts' gate and up projections (large: an
    expert's output outweighs the stream, and a row whose choice flips under a two-byte type's rounding is lost)."""
    from safetensors.torch import load_file, save_file
    from machserve_amd.weights import write_random_model
    out = os.path.join(str(tmp), f"befirax_{name}_{seed}_{sharpen}_{experts}")
    write_random_model(dict(CONFIGS_ALL[name]), seed, out, dtype)
    path = os.path.join(out, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        t = w[k].float()
        if k == "embed":
            t = t * 40.0
        elif k.endswith((".mix.q", ".mix.k")):
            t = t * sharpen
        elif k.endswith((".up", ".gate")):
            t = t * experts
        elif k.endswith((".mix.in", ".mix.v", ".mix.dkv", ".mix.uk", ".mix.uv", ".mix.g")):
            t = t * 8.0
        elif k.endswith(".correction"):
            t = t * 10.0
        elif k.endswith((".lq1", ".lk2")):
            t = t * 1.5
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
    """What a run keeps in its element type: operands of matrix products and the embedding (not filters, not the router,
    not the streams' small tensors)."""
    if name.endswith((".conv", ".router", ".mix")) or ".hc" in name or t.dim() < 2:
        return False
    return True


def within(got: torch.Tensor, want: torch.Tensor, dtype) -> bool:
    """float32: every row within rounding of sums taken in another order (a key too many or too few, a window one token
    off or a state that is lost is off by 1e-2 and more).  bfloat16: rounding of activations grows through the layers, so
    half the rows must be within 4e-2; and where two router scores lie within that rounding of each other a row takes
    another expert than the plain model does, which moves that row by as much as the expert matters and the rows after it
    by a little: at most one row in thirty may be beyond 0.25 (logits that have nothing to do with the wanted ones are
    off by 1.4 in every row)."""
    e = relative_errors(got, want)
    if dtype == torch.float32:
        return float(e.max()) < 1e-4
    return float(e.median()) < 4e-2 and int((e > 0.25).sum()) <= max(1, e.numel() // 30)
