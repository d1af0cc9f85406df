"""Configuration of the Migurax decoder: layers with the norm after the sum, whose mixer is either a matrix-memory
recurrence (``mlstm``) or attention over a cached latent (``latent_attention``), and whose feed-forward is dense,
routed over experts, or absent.

``config.json`` keys: ``architecture`` (``"Migurax"``), ``vocab``, ``width``, ``norm.eps``, ``postln_alpha`` and ``layers``,
a list with one entry per layer: ``type`` (the mixer), ``mixer`` (its sizes and constants) and ``mlp`` (``kind`` ``dense``
with ``ff``, or ``moe`` with ``expert.ff``, ``router.experts`` and ``router.top``, or null).  Tensor names: ``embed``,
``head``, ``final.norm``, and below ``l<i>.``: ``norm1``, ``norm2``, ``mix.*``, ``mlp.*``.  The design names no greatest
position; ``max_positions`` is an optional key of this reader for the engine's own bookkeeping.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import (BlockSpec, ConfigError, DenseFFSpec, LatentAttentionSpec, MLSTMSpec, ModelConfig, ModelSpec, PairRotarySpec,
                   PostNormBlockSpec, RMSNormSpec, RoutedExpertsSpec, RunEntry)

MIXER_KEYS = {
    "mlstm": ("heads", "dim", "vdim", "gate_cap"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"),
}


def _positive_int(where: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"Migurax: {where} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class MiguraxConfig(ModelConfig):
    architecture: ClassVar[str] = "Migurax"

    vocab: int
    width: int
    layers: list
    norm: dict
    postln_alpha: float = 1.0
    max_positions: int = 1 << 17
    torch_dtype: str = ""

    def validate(self) -> None:
        _positive_int("vocab", self.vocab)
        _positive_int("width", self.width)
        _positive_int("max_positions", self.max_positions)
        if not isinstance(self.norm, dict) or not float(self.norm.get("eps", 0)) > 0:
            raise ConfigError("Migurax: norm.eps must be a positive number")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("Migurax: 'layers' must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"Migurax: layer {i} has mixer type {kind!r}; built: {', '.join(sorted(MIXER_KEYS))}")
            mixer = layer.get("mixer")
            missing = [k for k in MIXER_KEYS[kind] if not isinstance(mixer, dict) or k not in mixer]
            if missing:
                raise ConfigError(f"Migurax: layer {i} ({kind}) lacks mixer key(s): {', '.join(missing)}")
            for k in ("heads", "dim", "vdim") + (("rot_dim", "kv_rank", "q_rank") if kind == "latent_attention" else ()):
                _positive_int(f"layer {i} mixer.{k}", mixer[k])
            if kind == "latent_attention":
                rot = mixer["rot"]
                if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
                    raise ConfigError(f"Migurax: layer {i} mixer.rot needs 'base' and 'dims'")
                if rot["dims"] % 2 or not 0 < rot["dims"] <= mixer["rot_dim"]:
                    raise ConfigError(f"Migurax: layer {i} rotates {rot['dims']} of {mixer['rot_dim']} dimensions: an even number within them")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                _positive_int(f"layer {i} mlp.ff", mlp.get("ff"))
            elif mlp.get("kind") == "moe":
                _positive_int(f"layer {i} mlp.expert.ff", (mlp.get("expert") or {}).get("ff"))
                router = mlp.get("router") or {}
                experts, top = _positive_int(f"layer {i} mlp.router.experts", router.get("experts")), _positive_int(f"layer {i} mlp.router.top", router.get("top"))
                if top > experts:
                    raise ConfigError(f"Migurax: layer {i} picks {top} of {experts} experts")
            else:
                raise ConfigError(f"Migurax: layer {i} has mlp kind {mlp.get('kind')!r}; built: dense, moe, or null")

    def _mixer(self, layer: dict):
        m, eps = layer["mixer"], float(self.norm["eps"])
        if layer["type"] == "mlstm":
            cap = m["gate_cap"]
            return MLSTMSpec(hidden=self.width, heads=m["heads"], dim=m["dim"], vdim=m["vdim"],
                             gate_cap=None if cap is None else float(cap), norm_eps=eps)
        return LatentAttentionSpec(hidden=self.width, heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                                   kv_rank=m["kv_rank"], q_rank=m["q_rank"], scale=float(m["scale"]), norm_eps=eps, sink=True,
                                   position=PairRotarySpec(dims=m["rot"]["dims"], base=float(m["rot"]["base"])))

    def _ffn(self, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        if mlp["kind"] == "dense":
            return DenseFFSpec(hidden=self.width, intermediate=mlp["ff"], activation="relu2", bias=True)
        return RoutedExpertsSpec(hidden=self.width, intermediate=mlp["expert"]["ff"], experts=mlp["router"]["experts"],
                                 top=mlp["router"]["top"], activation="relu2", router_bias=True)

    def to_spec(self) -> ModelSpec:
        norm = RMSNormSpec(dim=self.width, eps=float(self.norm["eps"]), weight_name="")
        blocks: list[BlockSpec] = []
        for layer in self.layers:
            ffn = self._ffn(layer)
            blocks.append(PostNormBlockSpec(mixer=self._mixer(layer), ffn=ffn, mixer_norm=norm, ffn_norm=norm if ffn is not None else None,
                                            mixer_name="mix", ffn_name="mlp", mixer_norm_name="norm1", ffn_norm_name="norm2",
                                            alpha=float(self.postln_alpha)))
        return ModelSpec(vocab_size=self.vocab, hidden=self.width, layers=tuple(blocks),
                         order=tuple(RunEntry(layer=i) for i in range(len(blocks))), final_norm=norm, tie_head=False,
                         max_positions=self.max_positions, embed_name="embed", final_norm_name="final.norm", head_name="head",
                         weight_suffix="", layers_format="l{}")

    def to_dict(self) -> dict[str, Any]:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": dict(self.norm),
             "postln_alpha": self.postln_alpha, "layers": [dict(layer) for layer in self.layers]}
        if self.max_positions != type(self).max_positions:
            d["max_positions"] = self.max_positions
        if self.torch_dtype:
            d["torch_dtype"] = self.torch_dtype
        return d
