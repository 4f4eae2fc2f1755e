"""Plain Kugalorn decoder: whole sequences, no cache, one function per mechanism.

Several residual streams (hyper-connections): each sublayer reads a weighted sum of the streams and
writes back into all of them through a mixing matrix.  Mixers: grouped sliding-window attention with
unit-norm queries and keys and a linear distance penalty per head, and latent attention (keys and
values expanded from one narrow latent row a token plus one rotated key part shared by the heads)
with a sigmoid gate per head.  Feed-forward: experts with clamped gate and up behind a softmax-of-
the-chosen router with a bias, plus a shared expert.  A stretch of the layers may run several times.

Everything runs on the CPU in float64 from a configuration (the dict of config.json) and a dict of
tensors by checkpoint name.  Nothing of the product package is imported.

`rnd`: where given, applied to the activations that an engine with bfloat16 activations keeps in
bfloat16 between two operations; norms, scores, routers and the residual streams stay exact.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _same(t):
    return t


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


# ------------------------------------------------------------------------ small functions
def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight lies around zero: unit_rms(x) * (1 + w)."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    """RMS norm with the weight as stored."""
    return unit_rms(x, eps) * w


def head_slopes(H):
    """slope of head h = 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F64)


def rotate_pairs(x, positions, base, dims):
    """Rotation of neighbouring pairs (2i, 2i + 1) of the first `dims` entries of the last axis by the angle
    position * base^(-2i / dims); the rest passes.  x [T, ..., n], positions [T]."""
    T = x.shape[0]
    out = x.clone()
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = positions.to(F64)[:, None] * f[None, :]                      # [T, half]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------------------ mixers
def window_attention(n, W, m, eps, rnd=_same):
    """Grouped attention over the last mask.size positions (the token itself among them); q and k are scaled
    to unit root mean square per head; score = q.k * scale - slope_h * (i - j).  n [T, d]."""
    T = n.shape[0]
    H, G, dk, dv, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"]
    size = (m.get("mask") or {}).get("size") or T + 1          # no mask: every earlier position
    q = rnd(unit_rms(rnd(n @ W["q"].T).view(T, H, dk), eps))
    k = rnd(unit_rms(rnd(n @ W["k"].T).view(T, G, dk), eps))
    v = rnd(n @ W["v"].T).view(T, G, dv)
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).to(F64)
    seen = (dist >= 0) & (dist < size)
    slopes = head_slopes(H)
    out = torch.zeros(T, H, dv, dtype=n.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale - slopes[h] * dist
        s = s.masked_fill(~seen, -math.inf)
        p = torch.softmax(s, -1)
        out[:, h] = rnd(p) @ v[:, g]
    return rnd(out.reshape(T, H * dv)) @ W["o"].T


def latent_attention(n, W, m, eps, rnd=_same):
    """Causal attention whose keys and values come from a latent row c = norm(first kv_rank rows of W_dkv n)
    and one rotated key part (the last rot_dim rows of W_dkv n) that all heads share; a head's query is
    [dim plain, rot_dim rotated]; the head's output is gated by sigmoid(W_g n)."""
    T = n.shape[0]
    H, dk, dr, dv, r, scale = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    pos = torch.arange(T)
    q = rnd(n @ W["q"].T).view(T, H, dk + dr)
    q_plain, q_rot = q[..., :dk], rnd(rotate_pairs(q[..., dk:], pos, base, dims))
    ckr = rnd(n @ W["dkv"].T)
    c = rnd(plain_norm(ckr[:, :r], W["dkv.norm"], eps))
    k_rot = rnd(rotate_pairs(ckr[:, r:], pos, base, dims))            # [T, dr]
    k_plain = rnd(c @ W["uk"].T).view(T, H, dk)
    v = rnd(c @ W["uv"].T).view(T, H, dv)
    gate = torch.sigmoid(n @ W["g"].T)                                 # [T, H]
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, dv, dtype=n.dtype)
    for h in range(H):
        s = (q_plain[:, h] @ k_plain[:, h].T + q_rot[:, h] @ k_rot.T) * scale
        s = s.masked_fill(~causal, -math.inf)
        out[:, h] = (rnd(torch.softmax(s, -1)) @ v[:, h]) * gate[:, h:h + 1]
    return rnd(out.reshape(T, H * dv)) @ W["o"].T


# ------------------------------------------------------------------------ feed-forward
def clamped_expert(n, gate, up, down, limit, rnd=_same):
    """g = min(W_gate n, limit), u = clamp(W_up n, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(n @ gate.T, max=limit)
    u = torch.clamp(n @ up.T, -limit, limit)
    return rnd(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(n, router, bias, top):
    """The `top` largest logits of W n + b a token (the lower index wins a tie) and the softmax over them."""
    z = n @ router.T + bias
    order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), -1), z


def experts(n, W, spec, rnd=_same, margins_out=None):
    """Weighted sum of the chosen experts' outputs plus the shared expert (where there is one).
    margins_out: a list that receives, per token, how far the last chosen logit lies above the first one left
    out, as a share of the root mean square of all the sequence's logits about their mean (with two experts a
    token's own spread is the margin itself); infinite where all experts are chosen."""
    E, top = spec["router"]["experts"], spec["router"]["top"]
    limit = spec["expert"]["limit"]
    ids, wts, z = route(n, W["router"], W["router.b"], top)
    if margins_out is not None:
        zs = torch.sort(z, dim=-1, descending=True).values
        spread = (z - z.mean()).pow(2).mean().sqrt().clamp_min(1e-30)
        margins_out.append((zs[:, top - 1] - zs[:, top]) / spread if top < E else torch.full((n.shape[0],), math.inf, dtype=n.dtype))
    out = torch.zeros(n.shape[0], W["e0.down"].shape[0], dtype=n.dtype)
    for t in range(n.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += wts[t, j] * clamped_expert(n[t:t + 1], W[f"e{e}.gate"], W[f"e{e}.up"], W[f"e{e}.down"], limit, rnd)[0]
    if spec.get("shared") is not None:
        out = out + clamped_expert(n, W["shared.gate"], W["shared.up"], W["shared.down"], spec["shared"]["limit"], rnd)
    return out


# ------------------------------------------------------------------------------- model
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_order(cfg):
    """The layer indices in the order they run: layers start .. stop - 1 `times` times in a row, then the rest."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def hyper_step(xs, hc, fn, norm_w, eps, rnd=_same):
    """One sublayer over the streams xs [s, T, d]: u = sum_s in[s] x_s; y = fn(norm(u));
    x_t <- sum_s mix[s, t] x_s + out[t] y, all streams from the old ones."""
    u = torch.einsum("s,std->td", hc["in"], xs)
    y = fn(rnd(offset_norm(u, norm_w, eps)))
    return torch.einsum("sr,std->rtd", hc["mix"], xs) + hc["out"][:, None, None] * y[None]


def plain_step(x, fn, norm_w, eps, rnd=_same):
    """One sublayer over a single residual stream: x <- x + fn(norm(x))."""
    return x + fn(rnd(offset_norm(x, norm_w, eps)))


def forward(cfg, weights, tokens, rnd=_same, layer_outputs=None, margins_out=None):
    """Logits [T, vocab] of a whole sequence.  weights: tensors by checkpoint name (any float type).
    layer_outputs: a list that receives the residual stream (the sum of the streams) after every layer run.
    margins_out: see experts().  Without 'streams' in the configuration the model keeps one stream and adds."""
    weights = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    x = weights["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = x if S is None else torch.stack([x] * S)
    for i in layer_order(cfg):
        layer, W = cfg["layers"][i], sub(weights, f"l{i}.")
        m = layer["mixer"]
        attend = window_attention if layer["type"] == "attention" else latent_attention
        mix = lambda h: attend(h, sub(W, "mix."), m, eps, rnd)
        ff = lambda h: experts(h, sub(W, "mlp."), layer["mlp"], rnd, margins_out)
        if S is None:
            xs = plain_step(xs, mix, W["norm1"], eps, rnd)
            if layer.get("mlp") is not None:
                xs = plain_step(xs, ff, W["norm2"], eps, rnd)
        else:
            xs = hyper_step(xs, sub(W, "hc1."), mix, W["norm1"], eps, rnd)
            if layer.get("mlp") is not None:
                xs = hyper_step(xs, sub(W, "hc2."), ff, W["norm2"], eps, rnd)
        if layer_outputs is not None:
            layer_outputs.append(xs if S is None else xs.sum(0))
    x = xs if S is None else xs.sum(0)
    return rnd(offset_norm(x, weights["final.norm"], eps)) @ weights["head"].T
