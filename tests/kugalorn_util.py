"""Helpers of the Kugalorn tests: small configurations, weights that make every mechanism loud, folders."""
from __future__ import annotations

import json
import math
import os

import torch


def attn(heads, kv_heads, dim, vdim, scale, window=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, dims=None):
    return {"type": "latent_attention",
            "mixer": dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, scale=scale,
                          rot={"base": base, "dims": rot_dim if dims is None else dims})}


def moe(experts, top, ff, limit, shared=None, shared_limit=None):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        out["shared"] = {"ff": shared, "limit": shared_limit}
    return out


def layer(mixer: dict, mlp=None) -> dict:
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, streams=None, loop=None, eps=1e-5) -> dict:
    out = {"architecture": "Kugalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# Configurations that differ in every size and option: values as wide as keys and not, grouped heads, one head and a
# kv head a query head, windows of 2 to beyond the sequence, rotated parts wider and narrower than the plain part with
# fewer channels turning than the part holds, one to four streams and a model without the key (one stream, plain sums),
# a looped stretch at the start, in the middle, of one pass, and none, one to all experts chosen, with and without a
# shared expert, layers without a feed-forward, sizes that are no multiples of 8.
# K_MIXED chooses all its experts, so no discrete choice can turn under bfloat16 rounding and long bfloat16 runs count
# to their end; fewer than all are chosen in K_WIDE, K_ODD, K_PLAIN and the expert layer alone.
K_MIXED = config(64, 211, [
    layer(attn(4, 2, 16, 24, 0.3, window=20), moe(4, 4, 40, 0.8, shared=24, shared_limit=1.2)),
    layer(latent(2, 16, 8, 24, 32, 0.2), moe(4, 4, 40, 0.8, shared=24, shared_limit=1.2)),
    layer(attn(2, 1, 32, 32, 0.15, window=7), None),
    layer(latent(3, 8, 12, 16, 24, 0.25, base=500.0, dims=8), moe(3, 3, 16, 2.0)),
], streams=2, loop=(1, 3, 2))
K_WIDE = config(96, 333, [
    layer(latent(4, 24, 16, 8, 48, 0.12, base=50000.0), moe(5, 2, 24, 1.0, shared=16, shared_limit=0.7)),
    layer(attn(3, 3, 40, 40, 0.1, window=300), moe(5, 1, 24, 1.5)),
    layer(attn(6, 2, 8, 72, 0.5, window=33), None),
    layer(latent(1, 40, 24, 40, 40, 0.1, dims=10), moe(6, 3, 16, 1.0, shared=40, shared_limit=3.0)),
], streams=4)
K_ODD = config(52, 97, [
    layer(attn(1, 1, 20, 12, 0.25, window=2), moe(2, 1, 12, 1.0, shared=4, shared_limit=1.0)),
    layer(latent(1, 12, 4, 20, 20, 0.3, dims=2), None),
    layer(attn(5, 5, 12, 20, 0.3), moe(3, 2, 30, 0.5)),
], streams=1, loop=(0, 2, 3), eps=1e-2)
K_PLAIN = config(48, 101, [
    layer(attn(2, 1, 24, 24, 0.2, window=16), moe(4, 2, 24, 1.0, shared=8, shared_limit=2.0)),
    layer(latent(2, 8, 8, 8, 16, 0.35), moe(4, 2, 24, 1.0)),
], loop=(1, 2, 1))
ONLY = {
    "attention": config(48, 101, [layer(attn(4, 2, 16, 8, 0.5, window=24))], streams=1),
    "attention_equal": config(64, 101, [layer(attn(2, 1, 64, 64, 0.125, window=100))], streams=3),
    "attention_unmasked": config(48, 101, [layer(attn(2, 2, 24, 24, 0.4))], streams=2),
    "latent": config(48, 101, [layer(latent(2, 16, 8, 24, 32, 0.6))], streams=3),
    "latent_wide": config(64, 101, [layer(latent(3, 24, 40, 16, 280, 0.3, dims=24))], streams=2),     # a cache row of 320
    # head counts and sizes on borders of 8 (the per-head products on the matrix cores), and a cache row of 160 with 24
    # heads to it (wide rows, more heads than one block of columns holds)
    "latent_eights": config(48, 101, [layer(latent(8, 16, 8, 24, 32, 0.5))], streams=2),
    "latent_many_heads": config(64, 101, [layer(latent(24, 16, 8, 8, 152, 0.4, dims=4))], streams=1),
    "streams": config(40, 101, [layer(attn(1, 1, 8, 8, 0.3, window=4)), layer(attn(1, 1, 8, 8, 0.3, window=4))], streams=4),
    "moe": config(48, 101, [layer(attn(1, 1, 8, 8, 0.3, window=8), moe(6, 2, 24, 0.9, shared=16, shared_limit=1.4))], streams=2),
    "moe_odd": config(44, 101, [layer(attn(1, 1, 8, 8, 0.3, window=8), moe(3, 2, 20, 0.9, shared=12, shared_limit=1.4))], streams=2),
}
CONFIGS = dict(mixed=K_MIXED, wide=K_WIDE, odd=K_ODD, plain=K_PLAIN, **{"only_" + k: v for k, v in ONLY.items()})


def make_weights(raw: dict, seed: int) -> dict:
    """bfloat16 tensors for a configuration, scaled so that every mechanism moves the logits: mixers and
    feed-forwards add about the stream's own size, the streams' tensors are far from the identity, norm weights
    spread around zero, the experts' clamps are reached, the router's bias is not small."""
    from tuff_amd.models.registry import build_model, config_from_dict
    g = torch.Generator().manual_seed(seed)
    model = build_model(config_from_dict(raw))
    S = raw.get("streams") or 1
    out = {}
    for d in model.weight_decls():
        name, shape = d.name, tuple(d.shape)
        n = lambda std=1.0, mean=0.0: mean + std * torch.randn(shape, generator=g)
        last = name.split(".")[-1]
        if name == "embed":
            t = n(1.0)
        elif name == "head":
            t = n(1.0 / math.sqrt(shape[1]))
        elif ".hc" in name:
            t = {"in": n(0.3, 1.0 / S), "out": n(0.3, 1.0)}.get(last)
            if t is None:
                t = torch.eye(S) * 0.8 + 0.25 * torch.randn(shape, generator=g)
        elif name.endswith("dkv.norm"):
            t = n(0.2, 1.0)
        elif last in ("norm1", "norm2", "norm"):
            t = n(0.2)                                           # stored around zero
        elif last == "b":
            t = n(0.7)                                           # the router's bias
        elif last == "router":
            t = n(3.0 / math.sqrt(shape[1]))
        elif last == "g":
            t = n(2.0 / math.sqrt(shape[1]))
        elif len(shape) == 2:
            t = n(1.3 / math.sqrt(shape[1]))
        else:
            t = n(0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(raw: dict, weights: dict, out_dir: str) -> str:
    from safetensors.torch import save_file
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(out_dir, "model.safetensors"))
    return out_dir
