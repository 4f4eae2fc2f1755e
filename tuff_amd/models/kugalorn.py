"""The Kugalorn decoder put together from parts.

x = embed[token]; the model keeps `streams` copies of the residual stream (hyper-connections: a sublayer
reads a weighted sum of them and writes back into all of them through a mixing matrix; without `streams`
in the configuration, one stream and plain residual sums).  Every layer is pre-norm with RMS norms whose
stored weight lies around zero (x / rms * (1 + w)); the mixers are grouped sliding-window attention with
unit-norm queries and keys, no position encoding and a distance penalty 2^(-8 (h + 1) / H) (i - j) per head,
and latent attention (one narrow cached row a token, a rotated key part shared by the heads, a sigmoid gate
per head); the feed-forward is a mixture of gated experts with clamped gate and up, g' sigmoid(1.702 g')
(u' + 1), behind a router with a bias whose weights are the softmax over the chosen logits, plus a shared
expert of the same form.  Layers loop.start .. loop.stop - 1 run loop.times times in a row on the same
tensors, each pass with a cache of its own.  Logits = head norm(sum of the streams).

Tensors: 'embed', 'head', 'final.norm'; layer i: 'l<i>.norm1', 'l<i>.norm2', 'l<i>.mix.*', 'l<i>.mlp.*'
(experts 'l<i>.mlp.e<k>.gate|up|down', 'l<i>.mlp.router', 'l<i>.mlp.router.b', 'l<i>.mlp.shared.gate|up|down'),
'l<i>.hc1.in|out|mix', 'l<i>.hc2.in|out|mix'.
"""
from __future__ import annotations

from ..config.kugalorn import KugalornConfig
from ..parts.attention import AttentionMixer
from ..parts.base import WeightDecl
from ..parts.block import HyperConnectionBlock, PreNormBlock
from ..parts.ffn import GatedMLP, MoE
from ..parts.latent import LatentAttentionMixer
from ..parts.norm import RMSNorm
from .decoder import DecoderModel, LayerRun

SLOPE_SPAN = 8.0            # head h's distance slope is 2^(-SLOPE_SPAN (h + 1) / H)
SWISH_ALPHA = 1.702         # the experts' gate is g sigmoid(SWISH_ALPHA g)


def _norm(cfg: KugalornConfig, name: str) -> RMSNorm:
    return RMSNorm(cfg.width, cfg.eps, name, offset=1.0)


def _mixer(cfg: KugalornConfig, i: int):
    layer, d, p = cfg.layers[i], cfg.width, f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "attention":
        return AttentionMixer(d, m["heads"], m["kv_heads"], m["dim"], value_dim=m["vdim"], scale=m["scale"],
                              qk_norm_eps=cfg.eps, window=(m.get("mask") or {}).get("size"), slope_span=SLOPE_SPAN,
                              names={k: p + k for k in ("q", "k", "v", "o")})
    rot = m.get("rot") or {"base": 1.0, "dims": 0}
    return LatentAttentionMixer(d, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], norm_eps=cfg.eps,
                                scale=m["scale"], rot_base=rot["base"], rot_dims=rot["dims"],
                                names={k: p + k for k in ("q", "dkv", "dkv.norm", "uk", "uv", "g", "o")})


def _feed_forward(cfg: KugalornConfig, i: int):
    spec, d, p = cfg.layers[i].get("mlp"), cfg.width, f"l{i}.mlp."
    if spec is None:
        return None
    E = spec["router"]["experts"]
    names = {"router": p + "router", "router.b": p + "router.b",
             "experts": [(f"{p}e{k}.gate", f"{p}e{k}.up", f"{p}e{k}.down") for k in range(E)]}
    shared = spec.get("shared")
    shared_ffn = None
    if shared is not None:
        shared_ffn = GatedMLP(d, shared["ff"], activation="swish_clamp", limit=shared["limit"], alpha=SWISH_ALPHA,
                              names={k: f"{p}shared.{k}" for k in ("gate", "up", "down")})
    return MoE(d, E, spec["router"]["top"], spec["expert"]["ff"], names=names, activation="swish_clamp", gated=True,
               limit=spec["expert"]["limit"], alpha=SWISH_ALPHA, router_weights="softmax", scale_input=False,
               shared=shared_ffn)


def build_kugalorn(cfg: KugalornConfig) -> DecoderModel:
    d = cfg.width
    blocks = []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(cfg, i)
        norm2 = _norm(cfg, f"l{i}.norm2") if ffn is not None else None
        if cfg.streams is None:
            blocks.append(PreNormBlock(_norm(cfg, f"l{i}.norm1"), _mixer(cfg, i), norm2, ffn))
        else:
            names = {f"{k}{q}": f"l{i}.hc{q}.{k}" for q in ("1", "2") for k in ("in", "out", "mix")}
            blocks.append(HyperConnectionBlock(cfg.streams, _norm(cfg, f"l{i}.norm1"), _mixer(cfg, i), norm2, ffn, names=names))
    runs = [LayerRun(i) for i in cfg.run_order()]              # every run has a cache of its own
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=d, embedding=WeightDecl("embed", (cfg.vocab, d), "normal"),
        blocks=blocks, final_norm=_norm(cfg, "final.norm"), head=WeightDecl("head", (cfg.vocab, d), "normal"),
        schedule=runs, max_positions=cfg.max_positions, pad_hidden=True, streams=cfg.streams)
