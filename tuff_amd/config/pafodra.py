"""Configuration of the Pafodra decoder: a list of parallel layers, each with one of three mixers
(softmax attention with a sink, an RWKV-style recurrence, a gated delta rule) and a dense or
mixture-of-experts feed-forward or none.

config.json is nested:
    architecture: "Pafodra"        vocab, width: ints        embedding: {scale}        norm: {eps}
    layers: [{type, mixer: {...sizes...}, mlp: {...} | null, weights_of: j (optional)}, ...]
        type "attention":      mixer {heads, kv_heads, dim, vdim, scale}
        type "wkv":            mixer {heads, dim}
        type "channel_delta":  mixer {heads, kv_heads, dim, vdim, conv}
        mlp {kind: "dense", ff}  |  {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff} (optional)}
A layer with weights_of: j runs layer j's tensors with a cache or state of its own.  Sizes that
config.json does not give (the ranks of the narrow projections) are read from the tensors' shapes
when a folder is loaded, and are kept in the configuration as `ranks` for models made from it.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Optional

from .base import ConfigError, ModelConfig

MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
    "wkv": ("heads", "dim"),
    "channel_delta": ("heads", "kv_heads", "dim", "vdim", "conv"),
}
DEFAULT_RANKS = {"w": 32, "a": 32, "g": 32}       # for models made from a configuration alone


@dataclasses.dataclass
class PafodraConfig(ModelConfig):
    architecture: ClassVar[str] = "Pafodra"
    ignored: ClassVar[frozenset[str]] = ModelConfig.ignored | frozenset({"architecture"})

    vocab: int
    width: int
    layers: list
    embedding: dict = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-5})
    ranks: Optional[dict] = None          # {"l<i>": {"w": r} | {"a": r, "g": r}}: inner sizes of the narrow projections
    max_positions: Optional[int] = None

    def validate(self) -> None:
        self._int("vocab")
        self._int("width")
        if not isinstance(self.embedding, dict) or not isinstance(self.embedding.get("scale"), (int, float)):
            raise ConfigError("embedding.scale must be a number")
        if not isinstance(self.norm, dict) or not isinstance(self.norm.get("eps"), (int, float)) or not self.norm["eps"] > 0:
            raise ConfigError("norm.eps must be a positive number")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_KEYS:
                raise ConfigError(f"{where}.type must be one of {sorted(MIXER_KEYS)}")
            m = layer.get("mixer")
            need = MIXER_KEYS[layer["type"]]
            if not isinstance(m, dict) or any(k not in m for k in need):
                raise ConfigError(f"{where}.mixer lacks key(s): {', '.join(k for k in need if not isinstance(m, dict) or k not in m)}")
            for k in need:
                ok = isinstance(m[k], (int, float)) and m[k] > 0 if k == "scale" else isinstance(m[k], int) and not isinstance(m[k], bool) and m[k] >= 1
                if not ok:
                    raise ConfigError(f"{where}.mixer.{k} must be a positive {'number' if k == 'scale' else 'integer'}, got {m[k]!r}")
            if "kv_heads" in need and m["heads"] % m["kv_heads"]:
                raise ConfigError(f"{where}.mixer: heads {m['heads']} is no multiple of kv_heads {m['kv_heads']}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"{where}.mlp.kind must be 'dense' or 'moe' (or mlp null)")
                try:
                    if mlp["kind"] == "dense":
                        sizes = [mlp["ff"]]
                    else:
                        sizes = [mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]]
                        if mlp.get("shared") is not None:
                            sizes.append(mlp["shared"]["ff"])
                except (KeyError, TypeError) as e:
                    raise ConfigError(f"{where}.mlp lacks a key ({e})") from None
                if any(isinstance(v, bool) or not isinstance(v, int) or v < 1 for v in sizes):
                    raise ConfigError(f"{where}.mlp: sizes must be positive integers, got {sizes}")
                if mlp["kind"] == "moe" and mlp["router"]["top"] > mlp["router"]["experts"]:
                    raise ConfigError(f"{where}.mlp.router: top {mlp['router']['top']} of {mlp['router']['experts']} experts")
            j = layer.get("weights_of")
            if j is not None:
                if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(self.layers) or j == i:
                    raise ConfigError(f"{where}.weights_of must name another layer, got {j!r}")
                seen = {i}
                while self.layers[j].get("weights_of") is not None:          # a layer that itself runs another's tensors
                    seen.add(j)
                    j = self.layers[j]["weights_of"]
                    if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(self.layers) or j in seen:
                        raise ConfigError(f"{where}.weights_of leads to no layer with tensors of its own")
                if self.layers[j].get("type") != layer["type"]:
                    raise ConfigError(f"{where} uses the tensors of layer {j}, which is a '{self.layers[j].get('type')}' layer")

    # --------------------------------------------------------------------- derived
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs (its sizes are that layer's)."""
        while self.layers[i].get("weights_of") is not None:
            i = self.layers[i]["weights_of"]
        return i

    def rank(self, i: int, which: str) -> int:
        return int(((self.ranks or {}).get(f"l{i}") or {}).get(which, DEFAULT_RANKS[which]))

    def rank_tensors(self) -> dict:
        """{(layer key, which): tensor name whose first size is that rank}."""
        out = {}
        for i, layer in enumerate(self.layers):
            if layer.get("weights_of") is not None:
                continue
            if layer["type"] == "wkv":
                out[(f"l{i}", "w")] = f"l{i}.mix.w1"
            elif layer["type"] == "channel_delta":
                out[(f"l{i}", "a")] = f"l{i}.mix.a1"
                out[(f"l{i}", "g")] = f"l{i}.mix.g1"
        return out

    def with_shapes(self, shape_of) -> "PafodraConfig":
        """The configuration with the narrow projections' inner sizes as the checkpoint has them;
        shape_of(name) -> tuple, or None where the tensor is not there."""
        ranks = {k: dict(v) for k, v in (self.ranks or {}).items()}
        for (layer, which), name in self.rank_tensors().items():
            shape = shape_of(name)
            if shape is not None and len(shape) == 2:
                ranks.setdefault(layer, {})[which] = int(shape[0])
        return dataclasses.replace(self, ranks=ranks)

    def to_dict(self) -> dict[str, Any]:
        out = {"architecture": self.architecture}
        out.update(dataclasses.asdict(self))
        for k in ("ranks", "max_positions"):
            if out.get(k) is None:
                out.pop(k, None)
        return out
