"""Typed configuration of the Tobinex decoder, read from its config.json.

A Tobinex model is a list of layers, each with a mixer and an optional dense
feed-forward, normed AFTER each residual sum (the sublayers read the residual
stream itself), an embedding with a scale and an output head that is the
embedding table without that scale.  config.json names the architecture under
`architecture` and gives every size and every constant that differs between
models; tensors are `embed`, `final.norm` and, for layer i, `l<i>.norm1`,
`l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.*`.  Nothing is fixed in code but what
the design fixes; keys and values that are not implemented are refused, never
ignored.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Tuple

from .specs import (ConfigError, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerRun, LayerSpec, MixedHeadAttentionSpec,
                    ModelSpec, OnePlusRMSNormSpec)

ARCHITECTURE = "Tobinex"
MAX_POSITION = 1 << 20      # the engine's own bound on a context (block tables are made for it); the design has none


def _get(d, key, where):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json {where}{key}: missing")
    return d[key]


def _int(d, key, where, minimum=1):
    v = _get(d, key, where)
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json {where}{key}: expected an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json {where}{key}: must be >= {minimum}, got {v}")
    return v


def _float(d, key, where):
    v = _get(d, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json {where}{key}: expected a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class TobinexConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    postln_alpha: float
    layers: Tuple[dict, ...]        # as config.json gives them (checked)
    max_position: int = MAX_POSITION

    @classmethod
    def from_dict(cls, d: dict) -> "TobinexConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers: expected a list with at least one layer")
        eps = _float(_get(d, "norm", ""), "eps", "norm.")
        if not eps >= 0:
            raise ConfigError(f"config.json norm.eps: must be >= 0, got {eps}")
        cfg = cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""),
                  embedding_scale=_float(_get(d, "embedding", ""), "scale", "embedding."), norm_eps=eps,
                  postln_alpha=_float(d, "postln_alpha", ""), layers=tuple(copy.deepcopy(layers)),
                  max_position=_int(d, "max_position", "") if "max_position" in d else MAX_POSITION)
        cfg.model_spec()        # checks every layer
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "postln_alpha": self.postln_alpha, "layers": copy.deepcopy(list(self.layers))}
        if self.max_position != MAX_POSITION:
            d["max_position"] = self.max_position
        return d

    def _mixer(self, i: int, layer: dict):
        where = f"layers[{i}]."
        kind = _get(layer, "type", where)
        if kind != "attention":
            raise ConfigError(f"config.json {where}type: {kind!r} is not a mixer of this design (attention)")
        m = _get(layer, "mixer", where)
        where += "mixer."
        mask = m.get("mask") if isinstance(m, dict) else None
        window, keep_first = None, 0
        if mask is not None:
            window = _int(mask, "size", where + "mask.") if mask.get("size") is not None else None
            keep_first = _int(mask, "keep_first", where + "mask.", 0) if mask.get("keep_first") is not None else 0
        return MixedHeadAttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where),
            head_dim=_int(m, "dim", where), v_head_dim=_int(m, "vdim", where), scale=_float(m, "scale", where),
            qk_norm_eps=self.norm_eps, window=window, keep_first=keep_first if window is not None else 0,
            prefix=f"l{i}.mix.")

    def _feed_forward(self, i: int, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        where = f"layers[{i}].mlp."
        kind = _get(mlp, "kind", where)
        if kind != "dense":
            raise ConfigError(f"config.json {where}kind: {kind!r} is not a feed-forward of this design (dense)")
        return GatedMLPSpec(self.width, _int(mlp, "ff", where), "silu", f"l{i}.mlp.", names=("gate", "up", "down"))

    def model_spec(self) -> ModelSpec:
        layers = []
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json layers[{i}]: expected an object")
            parts = [("mixer_norm", OnePlusRMSNormSpec(self.width, self.norm_eps, f"l{i}.norm1", name="")),
                     ("mixer", self._mixer(i, layer))]
            ffn = self._feed_forward(i, layer)
            if ffn is not None:
                parts += [("ffn_norm", OnePlusRMSNormSpec(self.width, self.norm_eps, f"l{i}.norm2", name="")), ("ffn", ffn)]
            layers.append(LayerSpec(parts=tuple(parts), block="post_norm" if ffn is not None else "post_norm_mixer",
                                    residual_scale=self.postln_alpha))
        return ModelSpec(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, max_position=self.max_position,
            embedding=EmbeddingSpec(self.vocab, self.width, prefix="embed", scale=self.embedding_scale, name=""),
            layers=tuple(layers), order=tuple(LayerRun(i) for i in range(len(layers))),
            final_norm=OnePlusRMSNormSpec(self.width, self.norm_eps, "final.norm", name=""),
            head=HeadSpec(self.vocab, self.width, tied=True))
