"""Attention through a latent (`LatentAttentionSpec`).

    [cq' | c' | kr | gate] = W_in x                    one product over the concatenated rows (W_dq, W_dkv, W_g)
    cq = N(cq'),  c = N(c'),  kr rotated               the cache keeps ONE row [c | kr] a token
    q = W_uq cq                                        a head is [d unrotated | dr rotated]
    head h, position i, key j:  score = scale * (q_h[:d] . W_uk_h c_j + rot(q_h[d:]) . kr_j)
                                      = scale * ([W_uk_h^T q_h[:d] | rot(q_h[d:])] . [c_j | kr_j])
    o_h = (sum_j p_j c_j) W_uv_h^T * sigmoid(gate_h)   delta = W_o concat_h o_h

Keys and values are never expanded: every head's query is carried into the latent's space, the attention runs
over the cached rows with all heads reading the same one "key/value head" (a value being the first kv_rank
numbers of its key's row), and the result is carried back by W_uv.  The cache of a token is kv_rank + rot_dim
numbers whatever the number of heads.
"""
from __future__ import annotations

import torch

from ..cache.needs import KVNeed
from .base import ParamSpec, build_part, register
from .mixer import paged_attention


@register("mixer", "latent_attention")
class LatentAttention:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.position = build_part("position", spec.position, runtime)
        if getattr(self.position, "pairing", "interleaved") != "interleaved":
            raise ValueError("latent attention rotates interleaved pairs")
        self.w_in = self.w_uq = self.w_uk = self.w_uv_t = self.w_o = None
        self.q_norm = self.c_norm = None

    @staticmethod
    def _names(spec):
        return dict(zip(("dq", "dq_norm", "uq", "dkv", "dkv_norm", "uk", "uv", "gate", "o"), spec.names))

    @classmethod
    def params(cls, spec):
        n, s = cls._names(spec), spec
        p = {
            n["dq"]: ParamSpec((s.q_rank, s.hidden_size)),
            n["dq_norm"]: ParamSpec((s.q_rank,), "float", ("one_plus_normal", 0.05)),
            n["uq"]: ParamSpec((s.num_heads * (s.head_dim + s.rot_dim), s.q_rank)),
            n["dkv"]: ParamSpec((s.kv_rank + s.rot_dim, s.hidden_size)),
            n["dkv_norm"]: ParamSpec((s.kv_rank,), "float", ("one_plus_normal", 0.05)),
            n["uk"]: ParamSpec((s.num_heads * s.head_dim, s.kv_rank)),
            n["uv"]: ParamSpec((s.num_heads * s.v_head_dim, s.kv_rank)),
            n["o"]: ParamSpec((s.hidden_size, s.num_heads * s.v_head_dim)),
        }
        if s.output_gate:
            p[n["gate"]] = ParamSpec((s.num_heads, s.hidden_size))
        return p

    @classmethod
    def placement(cls, spec):
        n = cls._names(spec)
        return {n["dq_norm"]: "float32", n["dkv_norm"]: "float32"}

    @staticmethod
    def variants(spec, dtype):
        out = [("latent", None), ("attention_generic", None)]
        if dtype == "bfloat16" and spec.row % 16 == 0 and spec.row <= 256 and spec.num_heads <= 16:
            out.append(("attention_prefill", {"HEAD_DIM": spec.row}))
            out.append(("attention_decode", {"HEAD_DIM": spec.row, "GROUP": spec.num_heads}))
        return out

    def load(self, tensors):
        n, s = self._names(self.spec), self.spec
        rows = [tensors[n["dq"]], tensors[n["dkv"]]] + ([tensors[n["gate"]]] if s.output_gate else [])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        w_in = torch.cat(rows, dim=0)
        pad = -w_in.shape[0] % 16       # whole tiles of rows for the products (the few rows of the gate leave a rest)
        if pad:
            w_in = torch.cat([w_in, torch.zeros((pad, w_in.shape[1]), dtype=w_in.dtype, device=w_in.device)], dim=0)
        self.w_in = self.rt.weight(w_in.contiguous())
        self.w_uq = self.rt.weight(tensors[n["uq"]])
        self.w_o = self.rt.weight(tensors[n["o"]])
        act = self.rt.act_dtype
        self.w_uk = tensors[n["uk"]].to(act).contiguous()                                           # [heads d, rank]
        self.w_uv_t = tensors[n["uv"]].to(act).view(s.num_heads, s.v_head_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.q_norm, self.c_norm = tensors[n["dq_norm"]], tensors[n["dkv_norm"]]
        freq, dims = self.position.rotary_table()
        self.freq = freq if freq is not None else torch.zeros(1, dtype=torch.float32, device=self.rt.device)
        self.rot_dims = dims if freq is not None else 0
        self.magnitude = float(getattr(self.position, "magnitude", 1.0))

    @staticmethod
    def need_of(spec):
        """One row of kv_rank + rot_dim numbers a token, no value rows of their own."""
        return KVNeed(num_kv_heads=1, head_dim=spec.row, window=spec.window, page_size=spec.page_size, v_head_dim=0)

    def cache_need(self):
        return self.need_of(self.spec)

    def state_need(self):
        return None

    def forward(self, x, batch, cache, state=None):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        table = batch.block_tables[cache.group]
        act = rt.act_dtype
        proj = rt.linear(x, self.w_in, slabs=True)        # float32 [n, query latent | latent | rotated part | gate], maybe in slabs
        cq = ops.latent_prepare(proj, rt.empty((n, s.q_rank), act), cache.k, batch.positions, batch.seq_of_token, table,
                                s.q_rank, s.kv_rank, s.rot_dim, self.q_norm, self.c_norm, s.norm_eps, self.freq, self.rot_dims,
                                self.magnitude, write_kv=cache.writable)
        q = rt.linear(cq, self.w_uq, slabs=True)
        q_lat = ops.latent_absorb(q, self.w_uk, rt.empty((n, s.num_heads * s.row), act), batch.positions, self.freq,
                                  self.rot_dims, self.magnitude, s.num_heads, s.head_dim, s.rot_dim, s.kv_rank)
        fast = rt.dtype == "bfloat16" and s.row % 16 == 0 and s.row <= 256 \
            and ops.attention_fast_ok(s.num_heads, 1, cache.page_size, table.shape[1])
        if rt.dtype == "bfloat16" and not fast:
            rt.generic_attention_launches += 1      # the slow kernel class: a measurement must know it ran
        # the matrix-core kernels take values as wide as keys: the whole row is the value there, and the rotated
        # part's columns of the result are left unread
        width = s.row if fast else s.kv_rank
        lat = rt.empty((n, s.num_heads * width), act)
        paged_attention(rt, batch, q_lat, lat, cache.k, cache.k, cache.page_size, table, s.num_heads, 1, s.row, width,
                        s.scale, s.window, fast)
        out = ops.latent_expand(lat, self.w_uv_t, rt.empty((n, s.num_heads * s.v_head_dim), act), s.num_heads, s.kv_rank,
                                s.v_head_dim, gate=proj if s.output_gate else None, gate_at=s.q_rank + s.row)
        return rt.linear(out, self.w_o, slabs=True, defer=True)
