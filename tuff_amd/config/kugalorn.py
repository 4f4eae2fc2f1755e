"""Configuration of the Kugalorn decoder: pre-norm layers over several residual streams, each with a
sliding-window attention or a latent attention mixer and a mixture-of-experts feed-forward or none; a
stretch of the layers may run several times in a row.

config.json is nested:
    architecture: "Kugalorn"       vocab, width: ints       norm: {eps}
    streams: S (optional: without it the model keeps one residual stream and plain residual sums)
    loop: {start, stop, times} (optional: layers start .. stop - 1 run `times` times in a row)
    layers: [{type, mixer: {...}, mlp: {...} | null}, ...]
        type "attention":         mixer {heads, kv_heads, dim, vdim, scale, mask: {size}}
        type "latent_attention":  mixer {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims}}
        mlp {kind: "moe", router: {experts, top}, expert: {ff, limit}, shared: {ff, limit} (optional)}
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Optional

from .base import ConfigError, ModelConfig

MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"),
}


def _is_int(v, minimum=1) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v >= minimum


def _is_pos(v) -> bool:
    return isinstance(v, (int, float)) and not isinstance(v, bool) and v > 0


@dataclasses.dataclass
class KugalornConfig(ModelConfig):
    architecture: ClassVar[str] = "Kugalorn"
    ignored: ClassVar[frozenset[str]] = ModelConfig.ignored | frozenset({"architecture"})

    vocab: int
    width: int
    layers: list
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    streams: Optional[int] = None
    loop: Optional[dict] = None
    max_positions: Optional[int] = None

    def validate(self) -> None:
        self._int("vocab")
        self._int("width")
        if not isinstance(self.norm, dict) or not _is_pos(self.norm.get("eps")):
            raise ConfigError("norm.eps must be a positive number")
        if self.streams is not None:
            self._int("streams")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_KEYS:
                raise ConfigError(f"{where}.type must be one of {sorted(MIXER_KEYS)}")
            m = layer.get("mixer")
            need = MIXER_KEYS[layer["type"]]
            lacks = [k for k in need if not isinstance(m, dict) or k not in m]
            if lacks:
                raise ConfigError(f"{where}.mixer lacks key(s): {', '.join(lacks)}")
            for k in need:
                if not (_is_pos(m[k]) if k == "scale" else _is_int(m[k], 0 if k in ("dim", "rot_dim") else 1)):
                    raise ConfigError(f"{where}.mixer.{k} must be a positive {'number' if k == 'scale' else 'integer'}, got {m[k]!r}")
            if layer["type"] == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}.mixer: heads {m['heads']} is no multiple of kv_heads {m['kv_heads']}")
                mask = m.get("mask")
                if mask is not None and (not isinstance(mask, dict) or not _is_int(mask.get("size"))):
                    raise ConfigError(f"{where}.mixer.mask.size must be a positive integer")
            else:
                rot = m.get("rot")
                if m["rot_dim"] and (not isinstance(rot, dict) or not _is_pos(rot.get("base")) or not _is_int(rot.get("dims"), 0)):
                    raise ConfigError(f"{where}.mixer.rot must give base and dims")
                if m["rot_dim"] and (rot["dims"] % 2 or rot["dims"] > m["rot_dim"]):
                    raise ConfigError(f"{where}.mixer.rot.dims must be even and at most rot_dim, got {rot['dims']}")
                if m["dim"] + m["rot_dim"] < 1:
                    raise ConfigError(f"{where}.mixer: a head needs query channels")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    raise ConfigError(f"{where}.mlp.kind must be 'moe' (or mlp null)")
                try:
                    sizes = [mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]]
                    limits = [mlp["expert"]["limit"]]
                    if mlp.get("shared") is not None:
                        sizes.append(mlp["shared"]["ff"])
                        limits.append(mlp["shared"]["limit"])
                except (KeyError, TypeError) as e:
                    raise ConfigError(f"{where}.mlp lacks a key ({e})") from None
                if not all(_is_int(v) for v in sizes):
                    raise ConfigError(f"{where}.mlp: sizes must be positive integers, got {sizes}")
                if not all(_is_pos(v) for v in limits):
                    raise ConfigError(f"{where}.mlp: limits must be positive numbers, got {limits}")
                if mlp["router"]["top"] > mlp["router"]["experts"]:
                    raise ConfigError(f"{where}.mlp.router: top {mlp['router']['top']} of {mlp['router']['experts']} experts")
        if self.loop is not None:
            lp = self.loop
            ok = isinstance(lp, dict) and all(_is_int(lp.get(k), 0) for k in ("start", "stop")) and _is_int(lp.get("times"))
            if not ok or not 0 <= lp["start"] <= lp["stop"] <= len(self.layers):
                raise ConfigError(f"loop must give 0 <= start <= stop <= {len(self.layers)} and times >= 1, got {lp!r}")

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

    def run_order(self) -> list[int]:
        """The layers' indices in the order they run."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    def to_dict(self) -> dict[str, Any]:
        out = {"architecture": self.architecture}
        out.update(dataclasses.asdict(self))
        for k in ("streams", "loop", "max_positions"):
            if out.get(k) is None:
                out.pop(k, None)
        return out
