"""Several copies of the residual stream (hyper-connections): the part that says how one sublayer reads and
writes them, and the block arrangement built on it.

The residual stream of such a model is a float32 tensor [tokens, R, width].  Sublayer f with its norm N, its
coefficients a [R] (`in`), b [R] (`out`) and M [R, R] (`mix`, indexed [from, to]):

    u = sum_r a[r] X_r;   y = f(N(u));   X_t <- sum_r M[r, t] X_r + b[t] y     for every t, from the old rows

A write and the read that follows it are one kernel (`ops.streams_step`): a block hands its last result on as
`PendingWrite`, and the next block's first read (or the model's closing sum before the final norm) carries it
out, as the blocks with one stream hand on a delta that the next norm adds.
"""
from __future__ import annotations

import torch

from .base import ParamSpec, build_part, register


class PendingWrite:
    """A sublayer's result that is not yet written into the streams, and the coefficients to write it with."""
    __slots__ = ("delta", "connection")

    def __init__(self, delta, connection):
        self.delta, self.connection = delta, connection


@register("connection", "hyper")
class HyperConnection:
    graph_safe = True   # nothing is launched here: the block's kernels read the coefficients

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.read = self.out = self.mix = None

    @staticmethod
    def params(spec):
        if not spec.learned:
            return {}
        read, out, mix = spec.names
        r = spec.streams
        return {read: ParamSpec((r,), "float", ("one_plus_normal", 0.2)), out: ParamSpec((r,), "float", ("one_plus_normal", 0.2)),
                mix: ParamSpec((r, r), "float", ("eye_plus_normal", 0.1))}

    @staticmethod
    def placement(spec):
        """The coefficients enter the residual sums: float32 on the device (exact)."""
        return {name: "float32" for name in spec.names} if spec.learned else {}

    def load(self, tensors):
        r = self.spec.streams
        if self.spec.learned:
            read, out, mix = self.spec.names
            self.read, self.out, self.mix = tensors[read], tensors[out], tensors[mix]
        else:
            device = self.rt.device
            self.read = torch.ones(r, dtype=torch.float32, device=device)
            self.out = torch.ones(r, dtype=torch.float32, device=device)
            self.mix = torch.eye(r, dtype=torch.float32, device=device)


@register("block", "hyper_pre_norm")
class HyperPreNormBlock:
    """Pre-norm sublayers over several copies of the residual stream (see the module's head).  x is
    [tokens, R, width]; what comes in and goes out as `pending` is a `PendingWrite`."""

    roles = (("mixer_norm", "norm"), ("mixer_hc", "connection"), ("mixer", "mixer"),
             ("ffn_norm", "norm"), ("ffn_hc", "connection"), ("ffn", "feed_forward"))

    @staticmethod
    def variants(layer_spec, dtype):
        return [("streams", None)]

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def _read(self, x, pending, connection, norm):
        """Write what is pending, then the sublayer's normed input: one kernel."""
        rt = self.rt
        h = rt.empty((x.shape[0], x.shape[2]), rt.act_dtype)
        if pending is None:
            return rt.ops.streams_step(x, None, None, None, connection.read, norm.weight, norm.spec.eps, h)
        before = pending.connection
        return rt.ops.streams_step(x, rt.settle(pending.delta), before.mix, before.out, connection.read, norm.weight,
                                   norm.spec.eps, h)

    def forward(self, x, pending, batch, cache, state):
        if pending is not None and not isinstance(pending, PendingWrite):
            raise TypeError("a block over several streams follows a block with one")
        p = self.parts
        h = self._read(x, pending, p["mixer_hc"], p["mixer_norm"])
        pending = PendingWrite(self.mixer.forward(h, batch, cache, state), p["mixer_hc"])
        if "ffn" in p:
            h = self._read(x, pending, p["ffn_hc"], p["ffn_norm"])
            pending = PendingWrite(p["ffn"].forward(h, batch), p["ffn_hc"])
        return x, pending


@register("block", "hyper_pre_norm_mixer")
class HyperPreNormMixerBlock(HyperPreNormBlock):
    """The first half alone: a layer without a feed-forward."""

    roles = (("mixer_norm", "norm"), ("mixer_hc", "connection"), ("mixer", "mixer"))


def open_streams(rt, table, tokens, streams: int):
    """The streams at the start: every copy is the token's row of the embedding table."""
    return rt.ops.streams_open(table, tokens, rt.empty((tokens.numel(), streams, table.shape[1]), torch.float32))


def close_norm_streams(rt, x, pending, which, norm):
    """[rows, width] in the type the products read: the last write carried out without being stored, the sum of the copies
    RMS-normed by `norm` (the final norm), for the rows `which` names (None: every token in order).  One kernel."""
    ones = getattr(rt, "_stream_ones", None)
    if ones is None or ones.numel() < x.shape[1]:
        ones = rt._stream_ones = torch.ones(8, dtype=torch.float32, device=rt.device)
    rows = x.shape[0] if which is None else which.numel()
    h = rt.empty((rows, x.shape[2]), rt.act_dtype)
    if pending is None:
        return rt.ops.streams_step(x, None, None, None, ones[:x.shape[1]], norm.weight, norm.spec.eps, h, which=which, store=False)
    return rt.ops.streams_step(x, rt.settle(pending.delta), pending.connection.mix, pending.connection.out, ones[:x.shape[1]],
                               norm.weight, norm.spec.eps, h, which=which, store=False)


def close_streams(rt, x, pending, which):
    """float32 [rows, width]: the sum of the copies after the last write (not stored), for the rows `which` names
    (None: every token in order)."""
    rows = x.shape[0] if which is None else which.numel()
    out = rt.empty((rows, x.shape[2]), torch.float32)
    if pending is None:
        return rt.ops.streams_close(x, None, None, None, which, out)
    return rt.ops.streams_close(x, rt.settle(pending.delta), pending.connection.mix, pending.connection.out, which, out)
