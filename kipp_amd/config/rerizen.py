"""Typed configuration of the Rerizen decoder, read from its config.json.

A Rerizen model keeps `streams` copies of the residual stream (hyper-connections: every sublayer reads a weighted
sum of the copies and writes its result back into all of them) and is a list of pre-norm layers, each with one of
three mixers and an optional dense feed-forward:

    attention          grouped-query attention without rotation: biases on q, k and v, every head of q and k divided
                       by its root mean square, a factor on the query that grows with the position (`q_temp`), keys
                       and values of different sizes; `kv_from: j` reads layer j's keys and values
    latent_attention   keys and values made from a cached latent, a rotated key part shared by the heads
                       (interleaved pairs, frequencies stretched by the YaRN rule), a sliding window, a gate a head
    mlstm              the matrix memory of xLSTM with capped gate pre-activations

config.json names the architecture under `architecture` and gives every size and every constant that differs between
models; tensors are `embed`, `final.norm`, `head` and, for layer i, `l<i>.norm1`, `l<i>.norm2`, `l<i>.hc1.*`,
`l<i>.hc2.*`, `l<i>.mix.*`, `l<i>.mlp.*`.  Keys and values that are not implemented are refused, never ignored.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from .specs import (AttentionSpec, ConfigError, EmbeddingSpec, GatedMLPSpec, HeadSpec, HyperConnectionSpec,
                    LatentAttentionSpec, LayerRun, LayerSpec, MLSTMSpec, ModelSpec, NoPositionSpec, RMSNormSpec, RopeSpec,
                    ScaledRopeSpec)

ARCHITECTURE = "Rerizen"
MAX_POSITION = 1 << 20      # the engine's own bound on a context (block tables are made for it); the design has none
MIXERS = ("attention", "latent_attention", "mlstm")


def _get(d, key, where):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json {where}{key}: missing")
    return d[key]


def _int(d, key, where, minimum=1):
    v = _get(d, key, where)
    if isinstance(v, float) and v == int(v):
        v = int(v)
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


def _only(d, allowed, where):
    extra = sorted(set(d) - set(allowed))
    if extra:
        raise ConfigError(f"config.json {where}: {', '.join(extra)} not implemented (known: {', '.join(sorted(allowed))})")


@dataclass(frozen=True)
class RerizenConfig:
    vocab: int
    width: int
    norm_eps: float
    streams: Optional[int]
    logit_scale: float
    layers: Tuple[dict, ...]        # as config.json gives them (checked)
    max_position: int = MAX_POSITION

    @classmethod
    def from_dict(cls, d: dict) -> "RerizenConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers: expected a list with at least one layer")
        eps = _float(_get(d, "norm", ""), "eps", "norm.")
        if not eps >= 0:
            raise ConfigError(f"config.json norm.eps: must be >= 0, got {eps}")
        cfg = cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), norm_eps=eps,
                  streams=_int(d, "streams", "") if d.get("streams") is not None else None,
                  logit_scale=_float(d, "logit_scale", "") if d.get("logit_scale") is not None else 1.0,
                  layers=tuple(copy.deepcopy(layers)),
                  max_position=_int(d, "max_position", "") if "max_position" in d else MAX_POSITION)
        cfg.model_spec()        # checks every layer
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "logit_scale": self.logit_scale, "layers": copy.deepcopy(list(self.layers))}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.max_position != MAX_POSITION:
            d["max_position"] = self.max_position
        return d

    # -- mixers --------------------------------------------------------------------------------
    def _attention(self, i: int, m: dict, where: str):
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "q_temp", "kv_from"), where)
        q_temp = None
        if m.get("q_temp") is not None:
            q_temp = (_float(m["q_temp"], "coef", where + "q_temp."), _int(m["q_temp"], "every", where + "q_temp."))
        source = None
        if m.get("kv_from") is not None:
            source = _int(m, "kv_from", where, 0)
            if source >= i:
                raise ConfigError(f"config.json {where}kv_from: layer {source} is not an earlier layer")
        if source is not None and 0 <= source < len(self.layers) and isinstance(self.layers[source], dict) \
                and isinstance(self.layers[source].get("mixer"), dict):
            # a layer that reads another's keys and values may leave their sizes to that layer
            theirs = self.layers[source]["mixer"]
            m = dict({k: theirs[k] for k in ("kv_heads", "dim", "vdim") if k in theirs and k not in m}, **m)
        dim, vdim = _int(m, "dim", where), _int(m, "vdim", where)
        spec = AttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where), head_dim=dim,
            position=NoPositionSpec(), qk_norm_eps=self.norm_eps, scale=_float(m, "scale", where), prefix=f"l{i}.mix.",
            bias=True, qk_norm_weight=False, q_temp=q_temp, v_head_dim=vdim, own_kv=source is None,
            names=("q", "k", "v", "o", "q.norm", "k.norm"), bias_names=("q.b", "k.b", "v.b"))
        return spec, source

    def _latent(self, i: int, m: dict, where: str):
        _only(m, ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "rot", "mask"), where)
        rot_dim = _int(m, "rot_dim", where, 0)
        position = NoPositionSpec()
        if m.get("rot") is not None and rot_dim > 0:
            rot, at = m["rot"], where + "rot."
            _only(rot, ("base", "dims", "scaling"), at)
            dims = _int(rot, "dims", at)
            if dims > rot_dim:
                raise ConfigError(f"config.json {at}dims: {dims} exceeds rot_dim {rot_dim}")
            if rot.get("scaling") is not None:
                sc = rot["scaling"]
                _only(sc, ("factor", "original", "fast", "slow"), at + "scaling.")
                position = ScaledRopeSpec(head_dim=rot_dim, theta=_float(rot, "base", at), factor=_float(sc, "factor", at + "scaling."),
                                          original=_float(sc, "original", at + "scaling."), fast=_float(sc, "fast", at + "scaling."),
                                          slow=_float(sc, "slow", at + "scaling."), rotary_dim=dims, pairing="interleaved")
            else:
                position = RopeSpec(head_dim=rot_dim, theta=_float(rot, "base", at), rotary_dim=dims, pairing="interleaved")
        window = None
        if m.get("mask") is not None:
            _only(m["mask"], ("size",), where + "mask.")
            window = _int(m["mask"], "size", where + "mask.") if m["mask"].get("size") is not None else None
        return LatentAttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), head_dim=_int(m, "dim", where), rot_dim=rot_dim,
            v_head_dim=_int(m, "vdim", where), q_rank=_int(m, "q_rank", where), kv_rank=_int(m, "kv_rank", where),
            scale=_float(m, "scale", where), norm_eps=self.norm_eps, position=position, window=window, prefix=f"l{i}.mix.")

    def _mlstm(self, i: int, m: dict, where: str):
        _only(m, ("heads", "dim", "vdim", "gate_cap"), where)
        return MLSTMSpec(hidden_size=self.width, num_heads=_int(m, "heads", where), head_dim=_int(m, "dim", where),
                         v_head_dim=_int(m, "vdim", where), gate_cap=_float(m, "gate_cap", where), norm_eps=self.norm_eps,
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
        layers, order = [], []
        streams = self.streams if self.streams is not None else 1
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json layers[{i}]: expected an object")
            where = f"layers[{i}]."
            kind = _get(layer, "type", where)
            m = _get(layer, "mixer", where)
            if not isinstance(m, dict):
                raise ConfigError(f"config.json {where}mixer: expected an object")
            source = None
            if kind == "attention":
                mixer, source = self._attention(i, m, where + "mixer.")
            elif kind == "latent_attention":
                mixer = self._latent(i, m, where + "mixer.")
            elif kind == "mlstm":
                mixer = self._mlstm(i, m, where + "mixer.")
            else:
                raise ConfigError(f"config.json {where}type: {kind!r} is not a mixer of this design ({', '.join(MIXERS)})")
            if source is not None:
                theirs = layers[source].part("mixer")
                if not isinstance(theirs, AttentionSpec) or not theirs.own_kv:
                    raise ConfigError(f"config.json {where}mixer.kv_from: layer {source} keeps no keys and values of its own")
                if (theirs.num_kv_heads, theirs.head_dim, theirs.value_dim) != (mixer.num_kv_heads, mixer.head_dim, mixer.value_dim) \
                        or theirs.num_heads != mixer.num_heads:
                    raise ConfigError(f"config.json {where}mixer.kv_from: layer {source} has other head counts or sizes")
            learned = self.streams is not None
            parts = [("mixer_norm", RMSNormSpec(self.width, self.norm_eps, f"l{i}.norm1", name="")),
                     ("mixer_hc", HyperConnectionSpec(streams, f"l{i}.hc1.", learned=learned)), ("mixer", mixer)]
            ffn = self._feed_forward(i, layer)
            if ffn is not None:
                parts += [("ffn_norm", RMSNormSpec(self.width, self.norm_eps, f"l{i}.norm2", name="")),
                          ("ffn_hc", HyperConnectionSpec(streams, f"l{i}.hc2.", learned=learned)), ("ffn", ffn)]
            layers.append(LayerSpec(parts=tuple(parts), block="hyper_pre_norm" if ffn is not None else "hyper_pre_norm_mixer"))
            order.append(LayerRun(i, cache_of=source))
        return ModelSpec(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, max_position=self.max_position,
            embedding=EmbeddingSpec(self.vocab, self.width, prefix="embed", name=""),
            layers=tuple(layers), order=tuple(order),
            final_norm=RMSNormSpec(self.width, self.norm_eps, "final.norm", name=""),
            head=HeadSpec(self.vocab, self.width, tied=False, prefix="head", scale=self.logit_scale, name=""),
            streams=streams)
