"""Configuration of the Nebutar decoder: token embedding times a factor plus a learned position row; pre-norm layers (layer norm
with weight and bias) over ``streams`` copies of the residual joined by hyper-connections; a mixer of two mixers side by side
(``parallel``: attention without positions, soft-capped and masked to chunks, beside a gated delta rule); a feed-forward routed over
gated experts, the last few of which are the identity; a span of layers that runs several times in a row, each pass with a cache
of its own; the output head is the embedding table.

``config.json`` keys: ``architecture`` (``"Nebutar"``), ``vocab``, ``width``, ``max_positions``, ``norm.eps``, ``embedding.scale``,
``streams`` (absent: one plain residual), ``loop`` (``start``, ``stop``, ``times``; absent: every layer once) and ``layers``, one entry
per layer: ``type`` (the mixer), ``mixer`` (its sizes and constants) and ``mlp`` (``kind`` ``moe`` with ``expert.ff``, ``router.experts``,
``router.identity`` and ``router.top``, or null).  Tensor names: ``embed``, ``pos``, ``final.norm`` (+ ``.b``), and below ``l<i>.``:
``norm1``, ``norm2`` (+ ``.b``), ``hc1.*``, ``hc2.*``, ``mix.left.*``, ``mix.right.*``, ``mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar

from .base import (BlockSpec, CappedAttentionSpec, ConfigError, GatedDeltaSpec, HyperBlockSpec, LayerNormSpec, ModelConfig, ModelSpec,
                   ParallelMixerSpec, RoutedExpertsSpec, RunEntry)

LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
RIGHT_KEYS = ("heads", "kv_heads", "dim", "vdim", "conv")


def _positive_int(where: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"Nebutar: {where} must be a positive integer, got {v!r}")
    return v


def _number(where: str, v) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"Nebutar: {where} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class NebutarConfig(ModelConfig):
    architecture: ClassVar[str] = "Nebutar"

    vocab: int
    width: int
    layers: list
    norm: dict
    max_positions: int
    embedding: dict = field(default_factory=lambda: {"scale": 1.0})
    streams: int = 0
    loop: dict = field(default_factory=dict)
    torch_dtype: str = ""

    def validate(self) -> None:
        _positive_int("vocab", self.vocab)
        _positive_int("width", self.width)
        _positive_int("max_positions", self.max_positions)
        if not isinstance(self.norm, dict) or not _number("norm.eps", self.norm.get("eps")) > 0:
            raise ConfigError("Nebutar: norm.eps must be a positive number")
        if not isinstance(self.embedding, dict):
            raise ConfigError("Nebutar: 'embedding' must be an object with 'scale'")
        _number("embedding.scale", self.embedding.get("scale", 1.0))
        if self.streams:
            _positive_int("streams", self.streams)
            if self.streams > 8:
                raise ConfigError(f"Nebutar: hyper-connections are built for up to 8 streams, not {self.streams}")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("Nebutar: 'layers' must be a non-empty list")
        if self.loop:
            for k in ("start", "stop", "times"):
                if not isinstance(self.loop.get(k), int) or isinstance(self.loop.get(k), bool):
                    raise ConfigError(f"Nebutar: loop.{k} must be an integer")
            if not 0 <= self.loop["start"] <= self.loop["stop"] <= len(self.layers) or self.loop["times"] < 1:
                raise ConfigError(f"Nebutar: loop {self.loop} does not fit {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind != "parallel":
                raise ConfigError(f"Nebutar: layer {i} has mixer type {kind!r}; built: parallel")
            mixer = layer.get("mixer")
            for side, keys in (("left", LEFT_KEYS), ("right", RIGHT_KEYS)):
                m = mixer.get(side) if isinstance(mixer, dict) else None
                missing = [k for k in keys if not isinstance(m, dict) or k not in m]
                if missing:
                    raise ConfigError(f"Nebutar: layer {i} mixer.{side} lacks key(s): {', '.join(missing)}")
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(f"layer {i} mixer.{side}.{k}", m[k])
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"Nebutar: layer {i} mixer.{side}: {m['heads']} heads are not a multiple of {m['kv_heads']} key heads")
            _positive_int(f"layer {i} mixer.right.conv", mixer["right"]["conv"])
            _number(f"layer {i} mixer.left.scale", mixer["left"]["scale"])
            if mixer["left"].get("softcap") is not None and not _number(f"layer {i} mixer.left.softcap", mixer["left"]["softcap"]) > 0:
                raise ConfigError(f"Nebutar: layer {i} mixer.left.softcap must be positive")
            mask = mixer["left"].get("mask")
            if mask is not None:
                _positive_int(f"layer {i} mixer.left.mask.size", mask.get("size") if isinstance(mask, dict) else None)
            for k in ("left_scale", "right_scale"):
                _number(f"layer {i} mixer.{k}", mixer.get(k, 1.0))
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") != "moe":
                raise ConfigError(f"Nebutar: layer {i} has mlp kind {mlp.get('kind')!r}; built: moe, or null")
            _positive_int(f"layer {i} mlp.expert.ff", (mlp.get("expert") or {}).get("ff"))
            router = mlp.get("router") or {}
            experts, top = _positive_int(f"layer {i} mlp.router.experts", router.get("experts")), _positive_int(f"layer {i} mlp.router.top", router.get("top"))
            identity = router.get("identity", 0)
            if not isinstance(identity, int) or isinstance(identity, bool) or identity < 0:
                raise ConfigError(f"Nebutar: layer {i} mlp.router.identity must be a count, got {identity!r}")
            if top > experts + identity:
                raise ConfigError(f"Nebutar: layer {i} picks {top} of {experts + identity} experts")

    # ------------------------------------------------------------------ parts
    def _mixer(self, layer: dict) -> ParallelMixerSpec:
        m, eps = layer["mixer"], float(self.norm["eps"])
        left, right = m["left"], m["right"]
        cap = left.get("softcap")
        mask = left.get("mask") or {}
        attention = CappedAttentionSpec(hidden=self.width, heads=left["heads"], kv_heads=left["kv_heads"], dim=left["dim"], vdim=left["vdim"],
                                        scale=float(left["scale"]), softcap=None if cap is None else float(cap), chunk=mask.get("size"))
        delta = GatedDeltaSpec(hidden=self.width, heads=right["heads"], kv_heads=right["kv_heads"], dim=right["dim"], vdim=right["vdim"],
                               conv=right["conv"], norm_eps=eps)
        return ParallelMixerSpec(hidden=self.width, branches=(("left", attention, float(m.get("left_scale", 1.0))),
                                                              ("right", delta, float(m.get("right_scale", 1.0)))))

    def _ffn(self, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        r = mlp["router"]
        return RoutedExpertsSpec(hidden=self.width, intermediate=mlp["expert"]["ff"], experts=r["experts"], top=r["top"], activation="silu",
                                 router_bias=False, gated=True, scores="all", choice_bias=True, identity=r.get("identity", 0))

    def run_order(self) -> list[int]:
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    def to_spec(self) -> ModelSpec:
        norm = LayerNormSpec(dim=self.width, eps=float(self.norm["eps"]), weight_name="", bias_name="b")
        names = dict(mixer_name="mix", ffn_name="mlp", mixer_norm_name="norm1", ffn_norm_name="norm2")
        blocks: list[BlockSpec] = []
        for layer in self.layers:
            ffn = self._ffn(layer)
            ffn_norm = norm if ffn is not None else None
            if self.streams:
                blocks.append(HyperBlockSpec(mixer=self._mixer(layer), ffn=ffn, mixer_norm=norm, ffn_norm=ffn_norm, streams=self.streams, **names))
            elif ffn is None:
                raise ConfigError("Nebutar: a layer without a feed-forward needs hyper-connections ('streams'); the plain pre-norm block has both sublayers")
            else:
                blocks.append(BlockSpec(mixer=self._mixer(layer), ffn=ffn, mixer_norm=norm, ffn_norm=ffn_norm, **names))
        return ModelSpec(vocab_size=self.vocab, hidden=self.width, layers=tuple(blocks),
                         order=tuple(RunEntry(layer=i) for i in self.run_order()), final_norm=norm, tie_head=True,
                         max_positions=self.max_positions, embed_name="embed", final_norm_name="final.norm", head_name="head",
                         embed_scale=float(self.embedding.get("scale", 1.0)), weight_suffix="", layers_format="l{}",
                         position_table_name="pos", streams=self.streams)

    def to_dict(self) -> dict[str, Any]:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
             "norm": dict(self.norm), "embedding": dict(self.embedding), "layers": [dict(layer) for layer in self.layers]}
        if self.streams:
            d["streams"] = self.streams
        if self.loop:
            d["loop"] = dict(self.loop)
        if self.torch_dtype:
            d["torch_dtype"] = self.torch_dtype
        return d
