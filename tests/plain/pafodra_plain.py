"""Plain Pafodra decoder: whole sequences, no cache, one function per mechanism.

A Pafodra layer is parallel: with n = dyt(x), x <- x + mixer(n) + feed_forward(n).  The mixers are
softmax attention with a sink and no position encoding, an RWKV-style recurrence with per-channel
decay ("wkv"), and a gated delta rule with short convolutions ("channel_delta"); the feed-forwards a
gated dense layer with biases and a mixture of experts with a sigmoid router.

Everything runs on the CPU in float64 from a configuration (the dict of config.json) and a dict of
tensors by checkpoint name.  Nothing of the product package is imported.

`rnd`: where given, applied to the activations that an engine with bfloat16 activations keeps in
bfloat16 between two operations (the normed input, projections' outputs, convolution outputs,
what a second product takes); recurrences, norms, scores, routers and the residual stream stay exact.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def _same(t):
    return t


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


# ------------------------------------------------------------------------ small functions
def dyt(x, w, b, alpha):
    """Dynamic tanh: tanh(alpha x) w + b; no statistics of x."""
    return torch.tanh(alpha * x) * w + b


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------------------ mixers
def sink_attention(n, W, p, m, rnd=_same):
    """Causal softmax attention, grouped heads, no positions; each head's denominator also holds
    exp(sink_h).  n [T, d]; W: tensors 'q','k','v','o','sink'; m: the mixer's sizes."""
    T = n.shape[0]
    H, G, dk, dv, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"]
    q = rnd(n @ W["q"].T).view(T, H, dk)
    k = rnd(n @ W["k"].T).view(T, G, dk)
    v = rnd(n @ W["v"].T).view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=n.dtype)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~causal, -math.inf)
        sink = W["sink"][h]
        top = torch.maximum(s.max(-1).values, sink)
        e = torch.exp(s - top[:, None])
        den = e.sum(-1) + torch.exp(sink - top)
        out[:, h] = rnd(e / den[:, None]) @ v[:, g]
    return rnd(out.reshape(T, H * dv)) @ W["o"].T


def wkv(n, W, m, eps, rnd=_same):
    """Time mixing with a decaying matrix state per head.  Each of r, k, v, g, w reads its own
    blend of the token's input and the one before it."""
    T, d = n.shape
    H, D = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, d, dtype=n.dtype), n[:-1]])
    mix = {s: rnd(n + (prev - n) * W["mu." + s]) for s in "rkvgw"}
    r = rnd(mix["r"] @ W["r"].T).view(T, H, D)
    k = rnd(mix["k"] @ W["k"].T).view(T, H, D)
    v = rnd(mix["v"] @ W["v"].T).view(T, H, D)
    gate = rnd(silu(mix["g"] @ W["g"].T))
    lw = rnd(torch.tanh(mix["w"] @ W["w1"].T)) @ W["w2"].T + W["w0"]
    decay = torch.exp(-torch.exp(lw)).view(T, H, D)
    u = W["u"]
    S = torch.zeros(H, D, D, dtype=n.dtype)                 # [head, key channel, value channel]
    o = torch.zeros(T, H, D, dtype=n.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    o = unit_rms(o, eps).reshape(T, H * D) * W["norm"] * gate
    return rnd(o) @ W["o"].T


def causal_conv(x, taps):
    """y[t, c] = sum_j taps[c, j] x[t - (K-1) + j, c], zeros before the start; the last tap is the
    current token's."""
    T, C = x.shape
    K = taps.shape[1]
    xp = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x])
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + xp[j:j + T] * taps[:, j]
    return y


def channel_delta(n, W, m, eps, rnd=_same):
    """Gated delta rule with a decay per head and key channel."""
    T = n.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(silu(causal_conv(rnd(n @ W["q"].T), W["q.conv"]))).view(T, G, dk)
    k = rnd(silu(causal_conv(rnd(n @ W["k"].T), W["k.conv"]))).view(T, G, dk)
    v = rnd(silu(causal_conv(rnd(n @ W["v"].T), W["v.conv"]))).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(n @ W["b"].T)                                          # [T, H]
    a = rnd(n @ W["a1"].T) @ W["a2"].T + W["dt_bias"]
    g = torch.exp(-torch.exp(W["A_log"])[None, :, None] * softplus(a).view(T, H, dk))
    S = torch.zeros(H, dk, dv, dtype=n.dtype)
    o = torch.zeros(T, H, dv, dtype=n.dtype)
    rep = H // G
    for t in range(T):
        kt = k[t].repeat_interleave(rep, 0)
        qt = q[t].repeat_interleave(rep, 0)
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hij,hi->hj", S, kt))
        S = S + kt[:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hij,hi->hj", S, qt)
    gate = torch.sigmoid(rnd(n @ W["g1"].T) @ W["g2"].T).view(T, H, dv)
    o = unit_rms(o, eps) * W["norm"] * gate
    return rnd(o.reshape(T, H * dv)) @ W["o"].T


# ------------------------------------------------------------------------ feed-forwards
def dense_ff(n, W, rnd=_same):
    a = gelu_tanh(n @ W["gate"].T + W["gate.b"]) * (n @ W["up"].T + W["up.b"])
    return rnd(a) @ W["down"].T + W["down.b"]


def expert(x, up, down, rnd=_same):
    return rnd(torch.relu(x @ up.T) ** 2) @ down.T


def moe_ff(n, W, spec, rnd=_same, margins: list | None = None):
    """Sigmoid scores, the `top` largest chosen, their scores (not renormalised) multiply the
    experts' inputs; a shared expert for every token, gated by one sigmoid per token.
    margins: gets, per token, how far the last chosen logit lies above the first one left out, in units of
    the logits' spread (infinite where every expert is chosen): a small one is a close call, which rounding
    may decide the other way."""
    T, d = n.shape
    E, top = spec["router"]["experts"], spec["router"]["top"]
    z = n @ W["router"].T
    s = torch.sigmoid(z)
    if margins is not None:
        zs = torch.sort(z, dim=-1, descending=True).values
        gap = (zs[:, top - 1] - zs[:, top]) if top < E else torch.full((T,), math.inf, dtype=z.dtype)
        margins.append(gap / z.pow(2).mean().sqrt())
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    out = torch.zeros(T, d, dtype=n.dtype)
    for t in range(T):
        for e in order[t].tolist():
            out[t] += expert(rnd(s[t, e] * n[t]), W[f"e{e}.up"], W[f"e{e}.down"], rnd)
    if spec.get("shared") is not None:
        sg = torch.sigmoid(n @ W["shared.sg"].T)                                 # [T, 1]
        out = out + sg * expert(n, W["shared.up"], W["shared.down"], rnd)
    return out


# -------------------------------------------------------------------------------- model
def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens, rnd=_same, layers_out: list | None = None,
            margins_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its start.  layers_out: gets the residual stream after
    every layer run.  margins_out: gets the routers' margins [T] of every layer run with experts (moe_ff)."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        n = rnd(dyt(x, W[p + "norm1"], W[p + "norm1.b"], W[p + "norm1.alpha"]))
        mw, kind, m = sub(W, p + "mix."), layer["type"], layer["mixer"]
        if kind == "attention":
            y = sink_attention(n, mw, p, m, rnd)
        elif kind == "wkv":
            y = wkv(n, mw, m, eps, rnd)
        elif kind == "channel_delta":
            y = channel_delta(n, mw, m, eps, rnd)
        else:
            raise ValueError(f"unknown mixer {kind}")
        spec = layer.get("mlp")
        if spec is not None:
            fw = sub(W, p + "mlp.")
            y = y + (dense_ff(n, fw, rnd) if spec["kind"] == "dense" else moe_ff(n, fw, spec, rnd, margins_out))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    n = rnd(dyt(x, W["final.norm"], W["final.norm.b"], W["final.norm.alpha"]))
    return n @ W["head"].T


def load_folder(model_dir: str):
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name)
    return cfg, weights
