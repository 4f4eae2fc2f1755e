"""Helpers of the Pafodra tests: small configurations, weights that make every mechanism loud, folders."""
from __future__ import annotations

import json
import math
import os

import torch


def attn(heads, kv_heads, dim, vdim, scale):
    return {"type": "attention", "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)}


def wkv(heads, dim):
    return {"type": "wkv", "mixer": dict(heads=heads, dim=dim)}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "channel_delta", "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer: dict, mlp=None, weights_of=None) -> dict:
    out = dict(mixer, mlp=mlp)
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def config(width, vocab, layers, scale=3.0, eps=1e-5, ranks=None) -> dict:
    out = {"architecture": "Pafodra", "vocab": vocab, "width": width, "embedding": {"scale": scale},
           "norm": {"eps": eps}, "layers": layers}
    if ranks is not None:
        out["ranks"] = ranks
    return out


# Configurations that differ in every size and option: value widths equal to the keys' and not, grouped heads and
# one head, two to five taps, one to all experts chosen, with and without a shared expert, layers without a
# feed-forward, layers that run another layer's tensors (an attention layer and a recurrent one), head sizes
# above 64 (two blocks of value channels in the recurrence kernels), sizes that are no multiples of 8.
# P_MIXED chooses all its experts, so no discrete choice can turn under bfloat16 rounding and long bfloat16 runs
# count to their end; fewer than all are chosen in P_WIDE, P_ODD and the expert layer alone.
P_MIXED = config(64, 211, [
    layer(wkv(2, 16), dense(96)),
    layer(attn(4, 2, 16, 24, 0.3), moe(4, 4, 40, shared=24)),
    layer(delta(4, 2, 16, 8, 3), None),
    layer(attn(4, 2, 16, 24, 0.3), moe(4, 4, 40, shared=24), weights_of=1),
    layer(wkv(2, 16), dense(96), weights_of=0),
    layer(delta(2, 2, 24, 40, 2), moe(3, 3, 16)),
], ranks={"l0": {"w": 8}, "l2": {"a": 16, "g": 8}, "l5": {"a": 12, "g": 20}})
P_WIDE = config(96, 333, [
    layer(delta(2, 1, 40, 72, 5), dense(50)),
    layer(wkv(1, 80), moe(5, 1, 24, shared=10)),
    layer(attn(3, 3, 32, 32, 0.2), dense(128)),
    layer(attn(2, 1, 72, 8, 0.1), None),
], scale=2.0, eps=3e-4, ranks={"l0": {"a": 5, "g": 9}, "l1": {"w": 3}})
P_ODD = config(52, 97, [
    layer(attn(1, 1, 20, 12, 0.25), moe(2, 1, 12, shared=4)),
    layer(wkv(3, 12), None),
    layer(delta(3, 3, 12, 20, 4), dense(30)),
], scale=4.0, eps=1e-2, ranks={"l1": {"w": 6}, "l2": {"a": 4, "g": 4}})
ONLY = {
    "attention": config(48, 101, [layer(attn(4, 2, 16, 8, 0.35))]),
    "attention_equal": config(64, 101, [layer(attn(2, 1, 64, 64, 0.125))]),
    "wkv": config(48, 101, [layer(wkv(2, 24))], ranks={"l0": {"w": 8}}),
    "wkv_wide": config(48, 101, [layer(wkv(1, 144))], ranks={"l0": {"w": 8}}),          # a head of 144: three quarters of the widest form
    "delta": config(48, 101, [layer(delta(4, 2, 16, 24, 4))], ranks={"l0": {"a": 8, "g": 8}}),
    # one tap: the convolution keeps no tail; the second layer runs the first one's tensors on a state of its own
    "delta_one_tap": config(40, 101, [layer(delta(2, 1, 8, 12, 1)), layer(delta(2, 1, 8, 12, 1), weights_of=0)],
                            ranks={"l0": {"a": 8, "g": 16}}),
    "dense": config(48, 101, [layer(attn(1, 1, 8, 8, 0.3), dense(72))]),
    "moe": config(48, 101, [layer(attn(1, 1, 8, 8, 0.3), moe(6, 2, 24, shared=16))]),
}
CONFIGS = dict(mixed=P_MIXED, wide=P_WIDE, odd=P_ODD, **{"only_" + k: v for k, v in ONLY.items()})


def make_weights(raw: dict, seed: int, loud_attention: float = 1.0) -> dict:
    """bfloat16 tensors for a configuration, scaled so that every mechanism moves the logits: mixers and
    feed-forwards add about the stream's own size, decays spread over (0, 1), sinks hold a share of the
    weight, gates are not stuck, biases are not small.  loud_attention scales W_q and W_k (peaky attention:
    a lost or extra key shows)."""
    from tuff_amd.models.registry import build_model, config_from_dict
    g = torch.Generator().manual_seed(seed)
    model = build_model(config_from_dict(raw))
    out = {}
    for d in model.weight_decls():
        name, shape = d.name, tuple(d.shape)
        n = lambda std=1.0, mean=0.0: mean + std * torch.randn(shape, generator=g)
        last = name.split(".")[-1]
        if name in ("embed",):
            t = n(1.0)
        elif name == "head":
            t = n(1.0 / math.sqrt(shape[1]))
        elif last == "alpha":
            t = torch.rand(shape, generator=g) * 0.5 + 0.3
        elif ".mix.mu." in name:
            t = torch.rand(shape, generator=g)
        elif last in ("norm1", "norm") and len(shape) == 1:
            t = n(0.2, 1.0)
        elif name.endswith("norm1.b") or name == "final.norm.b":
            t = n(0.2)
        elif last == "conv":
            t = n(0.6)
        elif last == "w0":
            t = n(1.0, -1.0)
        elif last == "u":
            t = n(0.5)
        elif last == "A_log":
            t = n(0.7)
        elif last == "dt_bias":
            t = n(1.0)
        elif last == "sink":
            t = n(1.5)
        elif last == "b" and len(shape) == 1:
            t = n(0.5)                                         # biases of the dense feed-forward
        elif len(shape) == 2:
            gain = 1.0
            if _kind(raw, name) == "attention" and last in ("q", "k"):
                gain = 2.0 * loud_attention
            if last in ("w2", "a2", "g2"):
                gain = 2.0
            if last == "router":
                gain = 3.0
            t = n(gain / math.sqrt(shape[1]))
        else:
            t = n(0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def _kind(raw: dict, name: str) -> str:
    if not name.startswith("l"):
        return ""
    return raw["layers"][int(name[1:].split(".")[0])]["type"]


def write_folder(raw: dict, weights: dict, out_dir: str) -> str:
    from safetensors.torch import save_file
    os.makedirs(out_dir, exist_ok=True)
    disk = {k: v for k, v in raw.items() if k != "ranks"}        # the ranks are read from the tensors' shapes
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(disk, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(out_dir, "model.safetensors"))
    return out_dir


def scales(t: torch.Tensor, factor: float) -> torch.Tensor:
    return (t.float() * factor).to(t.dtype)
