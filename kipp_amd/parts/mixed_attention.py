"""The attention mixer whose softmax weights are mixed across heads (`MixedHeadAttentionSpec`).

    q = Wq x, k = Wk x, v = Wv x, gate = Wg x          one product over the concatenated rows
    q, k RMS-normed over their whole projection        (all heads of a token at once, plain weights)
    score_h(i, j) = scale q_h(i) . k_c(j) - r1_h ln(1 + r2_h (i - j)),  c = h // (heads / kv heads)
    i sees j <= i when i - j < window or j < keep_first
    p_h = exp(score_h) / (exp(sink_h) + sum_j exp(score_h))
    p'_h = sum_g mix[h, g] p_g;   o_h = sum_j p'_h v_c;   delta = Wo (o * sigmoid(gate))

No rotation: positions enter through the distance bias and the mask alone.  Keys (size `head_dim`) and values
(`v_head_dim`) lie in the paged cache; a window gives pages back as it passes them, except those that hold the
kept first keys.  Each of distance bias, sink, mixing and gate can be switched off in the spec.
"""
from __future__ import annotations

import torch

from ..cache.needs import KVNeed
from .base import ParamSpec, register


@register("mixer", "mixed_head_attention")
class MixedHeadAttention:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_in = self.w_o = None
        self.q_norm = self.k_norm = self.r1 = self.r2 = self.sink = self.mix = None

    @staticmethod
    def _names(spec):
        return dict(zip(("q", "k", "v", "o", "q_norm", "k_norm", "r1", "r2", "sink", "mix", "gate"), spec.names))

    @classmethod
    def params(cls, spec):
        n = cls._names(spec)
        p = {
            n["q"]: ParamSpec((spec.q_dim, spec.hidden_size)),
            n["k"]: ParamSpec((spec.kv_dim, spec.hidden_size)),
            n["v"]: ParamSpec((spec.v_dim, spec.hidden_size)),
            n["o"]: ParamSpec((spec.hidden_size, spec.out_dim)),
            n["q_norm"]: ParamSpec((spec.q_dim,), "float", ("one_plus_normal", 0.05)),
            n["k_norm"]: ParamSpec((spec.kv_dim,), "float", ("one_plus_normal", 0.05)),
        }
        if spec.distance_bias:
            p[n["r1"]] = ParamSpec((spec.num_heads,), "float", ("abs_normal", 1.0))
            p[n["r2"]] = ParamSpec((spec.num_heads,), "float", ("abs_normal", 0.2))
        if spec.sink:
            p[n["sink"]] = ParamSpec((spec.num_heads,), "float", ("normal", 1.0))
        if spec.head_mixing:
            p[n["mix"]] = ParamSpec((spec.num_heads, spec.num_heads), "float", ("normal", 0.4))
        if spec.output_gate:
            p[n["gate"]] = ParamSpec((spec.out_dim, spec.hidden_size))
        return p

    @classmethod
    def placement(cls, spec):
        """The numbers that enter scores, softmax and norms are widened to float32 on the device (exact)."""
        n = cls._names(spec)
        return {n[k]: "float32" for k in ("q_norm", "k_norm", "r1", "r2", "sink", "mix")}

    @staticmethod
    def variants(spec, dtype):
        """The plain kernels, and under bfloat16 the build of the matrix-core form for these sizes where it takes them
        (any page size that it takes: the engine's is not known here)."""
        from ..csrc import ops
        out = [("attention_mixed", None)]
        if dtype == "bfloat16" and ops.mixed_attention_fast_ok(spec.num_heads, spec.head_dim, spec.v_head_dim, spec.page_size or 16):
            out += [("attention_mixed_mfma", defines)
                    for defines in ops.mixed_attention_builds(spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.v_head_dim)]
        return out

    def load(self, tensors):
        n, s = self._names(self.spec), self.spec
        rows = [tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]] + ([tensors[n["gate"]]] if s.output_gate else [])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        # rows concatenated: one product serves q, k, v and the gate, which all read the same input
        self.w_in = self.rt.weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = self.rt.weight(tensors[n["o"]])
        self.q_norm, self.k_norm = tensors[n["q_norm"]], tensors[n["k_norm"]]
        if s.distance_bias:
            self.r1, self.r2 = tensors[n["r1"]], tensors[n["r2"]]
        if s.sink:
            self.sink = tensors[n["sink"]]
        if s.head_mixing:
            self.mix = tensors[n["mix"]]

    @staticmethod
    def need_of(spec):
        """What a mixer of this spec keeps per token, known without building it."""
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim, window=spec.window, page_size=spec.page_size,
                      v_head_dim=spec.v_head_dim, keep_first=spec.keep_first if spec.window is not None else 0)

    def cache_need(self):
        return self.need_of(self.spec)

    def state_need(self):
        return None

    def forward(self, x, batch, cache, state=None):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        table = batch.block_tables[cache.group]
        proj = rt.linear(x, self.w_in, slabs=True)           # float32 [n, q | k | v | gate], maybe in slabs
        q = ops.mixed_prepare(proj, rt.empty((n, s.q_dim), rt.act_dtype), cache.k, cache.v, batch.positions,
                              batch.seq_of_token, table, s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim,
                              self.q_norm, self.k_norm, s.qk_norm_eps, write_kv=cache.writable)
        out = rt.empty((n, s.out_dim), rt.act_dtype)
        gate_at = s.q_dim + s.kv_dim + s.v_dim
        if rt.dtype == "bfloat16" and getattr(rt, "mixed_attention_fast", True) \
                and ops.mixed_attention_fast_ok(s.num_heads, s.head_dim, s.v_head_dim, cache.page_size):
            items, n_items, row_splits, max_splits, workspace = self._items(batch)
            ops.mixed_attention_mfma(q, cache.k, cache.v, out, items, n_items, row_splits, max_splits,
                                     batch.q_start, batch.q_len, batch.ctx_len, table,
                                     s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim, s.scale, s.window or 0,
                                     s.keep_first, self.r1, self.r2, self.sink, self.mix, workspace,
                                     gate=proj if s.output_gate else None, gate_at=gate_at)
            return rt.linear(out, self.w_o, slabs=True, defer=True)
        if rt.dtype == "bfloat16":
            rt.generic_attention_launches += 1      # the slow kernel class: a measurement must know it ran
        ops.mixed_attention_plain(q, cache.k, cache.v, out, batch.positions, batch.seq_of_token, table,
                                  s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim, s.scale, s.window or 0,
                                  s.keep_first, self.r1, self.r2, self.sink, self.mix,
                                  gate=proj if s.output_gate else None, gate_at=gate_at)
        return rt.linear(out, self.w_o, slabs=True, defer=True)

    def _items(self, batch):
        """The item list of the matrix-core form: every entry's rows in tiles of 16, and where the tiles alone are too
        few workgroups to fill the GPU, each tile's keys in several runs (at least 128 keys a run, at most 16 runs).
        Made by the first layer of a geometry and kept while the batch object lives: a recorded step keeps its own,
        made for the longest context of its class (the kernels take the true lengths from the device)."""
        s, ops = self.spec, self.rt.ops
        key = ("mixed_attention_work", s.num_heads, s.v_head_dim, s.window, s.keep_first)
        work = batch.host.get(key)
        if work is None:
            rows_tile, keys_tile = ops.MIXED_ROWS, ops.MIXED_KEYS
            window, keep = s.window or 0, s.keep_first
            tiles = []
            for e, (n, ctx) in enumerate(zip(batch.host["q_len"], batch.host["ctx_len"])):
                for row0 in range(0, n, rows_tile):
                    rows = min(rows_tile, n - row0)
                    pos0 = ctx - n + row0
                    lo = max(0, pos0 - window + 1) if window else 0
                    kept = min(keep, lo) if window else 0
                    kept_tiles = (kept - 1) // keys_tile + 1 if kept > 0 else 0
                    first = max(lo // keys_tile, kept_tiles)
                    tiles.append((e, row0, rows, kept_tiles + (pos0 + rows - 1) // keys_tile - first + 1))
            want = -(-2 * ops.compute_units(self.rt.device) // len(tiles))
            entry, row0s, split, nsplits, row_splits = [], [], [], [], []
            for e, row0, rows, key_tiles in tiles:
                runs = max(1, min(16, key_tiles // 4, want))
                entry += [e] * runs
                row0s += [row0] * runs
                split += list(range(runs))
                nsplits += [runs] * runs
                row_splits += [runs] * rows
            most = max(nsplits)
            lists = batch.upload(entry, row0s, split, nsplits, row_splits)
            space = ops.mixed_attention_workspace(len(entry), batch.n_tokens, s.num_heads, s.v_head_dim, most, self.rt.device)
            work = (tuple(lists[:4]), len(entry), lists[4], most, space)
            batch.host[key] = work
        return work
