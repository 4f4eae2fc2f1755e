"""The Pafodra decoder put together from parts.

x = embed[token] * embedding.scale; every layer is parallel, x <- x + mixer(h) + ff(h) with h = dyt(x)
(one dynamic-tanh norm a layer, read by both); the mixers are attention with a sink per head and no
position encoding, the wkv recurrence and the gated delta rule; the feed-forwards a gated layer with
the tanh form of gelu and biases, or experts with squared relu behind a sigmoid router whose scores
multiply the experts' inputs, plus a gated shared expert.  A layer that names another with weights_of
runs that layer's block again on a cache or state of its own.  Logits = head dyt(x).

Tensors: 'embed', 'head', 'final.norm{,.b,.alpha}'; layer i: 'l<i>.norm1{,.b,.alpha}', 'l<i>.mix.*',
'l<i>.mlp.*' (experts 'l<i>.mlp.e<k>.up|down', 'l<i>.mlp.router', 'l<i>.mlp.shared.up|down|sg').
"""
from __future__ import annotations

from ..config.pafodra import PafodraConfig
from ..parts.attention import AttentionMixer
from ..parts.base import WeightDecl
from ..parts.block import ParallelBlock
from ..parts.ffn import GatedMLP, MoE
from ..parts.norm import DynamicTanh
from ..parts.recurrent import GatedDeltaMixer, WkvMixer
from .decoder import DecoderModel, LayerRun


def _norm(d: int, name: str) -> DynamicTanh:
    return DynamicTanh(d, names={"weight": name, "bias": name + ".b", "alpha": name + ".alpha"})


def _mixer(cfg: PafodraConfig, i: int):
    layer, d, p = cfg.layers[i], cfg.width, f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "attention":
        return AttentionMixer(d, m["heads"], m["kv_heads"], m["dim"], value_dim=m["vdim"], scale=m["scale"],
                              names={k: p + k for k in ("q", "k", "v", "o", "sink")})
    if layer["type"] == "wkv":
        names = {k: p + k for k in ("mu.r", "mu.k", "mu.v", "mu.g", "mu.w", "r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")}
        return WkvMixer(d, m["heads"], m["dim"], cfg.eps, names=dict(names, rank=cfg.rank(i, "w")))
    names = {k: p + k for k in ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "A_log", "a1", "a2", "dt_bias", "g1", "g2",
                                "norm", "o")}
    return GatedDeltaMixer(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], cfg.eps,
                           names=dict(names, a_rank=cfg.rank(i, "a"), g_rank=cfg.rank(i, "g")))


def _feed_forward(cfg: PafodraConfig, i: int):
    spec, d, p = cfg.layers[i].get("mlp"), cfg.width, f"l{i}.mlp."
    if spec is None:
        return None
    if spec["kind"] == "dense":
        return GatedMLP(d, spec["ff"], activation="gelu_tanh", bias=True,
                        names={k: p + k for k in ("gate", "up", "down", "gate.b", "up.b", "down.b")})
    E = spec["router"]["experts"]
    names = {"router": p + "router", "experts": [(f"{p}e{k}.up", f"{p}e{k}.down") for k in range(E)]}
    shared = spec.get("shared")
    if shared is not None:
        names.update({k: p + k for k in ("shared.up", "shared.down", "shared.sg")})
    return MoE(d, E, spec["router"]["top"], spec["expert"]["ff"], names=names, activation="relu2",
               router_weights="sigmoid", scale_input=True, shared_dim=shared["ff"] if shared is not None else 0)


def build_pafodra(cfg: PafodraConfig) -> DecoderModel:
    d = cfg.width
    blocks, block_of, runs = [], {}, []
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is None:
            block_of[i] = len(blocks)
            blocks.append(ParallelBlock(_norm(d, f"l{i}.norm1"), _mixer(cfg, i), _feed_forward(cfg, i)))
    for i in range(len(cfg.layers)):
        runs.append(LayerRun(block_of[cfg.owner(i)]))           # every run has a cache or state of its own
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=d, embedding=WeightDecl("embed", (cfg.vocab, d), "normal"),
        blocks=blocks, final_norm=_norm(d, "final.norm"), head=WeightDecl("head", (cfg.vocab, d), "normal"),
        schedule=runs, max_positions=cfg.max_positions, embedding_scale=float(cfg.embedding["scale"]), pad_hidden=True)
