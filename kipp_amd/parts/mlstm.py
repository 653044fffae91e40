"""The matrix memory of xLSTM as a mixer (`MLSTMSpec`): a recurrent layer whose state of fixed size lives in the
request's slot.

    [q | k | v | gate | zi | zf] = W_in x              one product over the concatenated rows
    per head, token after token:  li = cap tanh((zi + bi) / cap),  lf = logsigmoid(cap tanh((zf + bf) / cap))
                                  m' = max(lf + m, li);  S' = e^(lf + m - m') S + e^(li - m') k v^T;  n' alike with k
                                  o = S'^T (q / sqrt(d)) / (max(|n' . q / sqrt(d)|, e^(-m')) + 1e-6)
    delta = W_o (o / rms(o) per head * w * sigmoid(gate))

The recurrence, the gates and the norms run in float32 under either precision; the state is float32.  A prompt
portion walks its tokens in order inside one kernel launch, a single token is a walk of one step: the same kernel,
so a position's result does not depend on how the tokens were cut.
"""
from __future__ import annotations

import torch

from ..cache.needs import StateNeed
from .base import ParamSpec, register


@register("mixer", "mlstm")
class MLSTM:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_in = self.w_o = self.norm = self.bias_i = self.bias_f = None

    @staticmethod
    def _names(spec):
        return dict(zip(("q", "k", "v", "gate", "o", "norm", "i", "i_bias", "f", "f_bias"), spec.names))

    @classmethod
    def params(cls, spec):
        n, s = cls._names(spec), spec
        hd, hv = s.num_heads * s.head_dim, s.num_heads * s.v_head_dim
        return {
            n["q"]: ParamSpec((hd, s.hidden_size)), n["k"]: ParamSpec((hd, s.hidden_size)),
            n["v"]: ParamSpec((hv, s.hidden_size)), n["gate"]: ParamSpec((hv, s.hidden_size)),
            n["o"]: ParamSpec((s.hidden_size, hv)),
            n["norm"]: ParamSpec((hv,), "float", ("one_plus_normal", 0.05)),
            n["i"]: ParamSpec((s.num_heads, s.hidden_size)), n["i_bias"]: ParamSpec((s.num_heads,), "float", ("normal", 1.0)),
            n["f"]: ParamSpec((s.num_heads, s.hidden_size)), n["f_bias"]: ParamSpec((s.num_heads,), "float", ("one_plus_normal", 1.0)),
        }

    @classmethod
    def placement(cls, spec):
        n = cls._names(spec)
        return {n["norm"]: "float32", n["i_bias"]: "float32", n["f_bias"]: "float32"}

    @staticmethod
    def variants(spec, dtype):
        return [("mlstm", None)]

    def load(self, tensors):
        n = self._names(self.spec)
        rows = [tensors[n[k]] for k in ("q", "k", "v", "gate", "i", "f")]
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        w_in = torch.cat(rows, dim=0)
        pad = -w_in.shape[0] % 16       # whole tiles of rows for the products (the gates' few rows leave a rest)
        if pad:
            w_in = torch.cat([w_in, torch.zeros((pad, w_in.shape[1]), dtype=w_in.dtype, device=w_in.device)], dim=0)
        self.w_in = self.rt.weight(w_in.contiguous())
        self.w_o = self.rt.weight(tensors[n["o"]])
        self.norm, self.bias_i, self.bias_f = tensors[n["norm"]], tensors[n["i_bias"]], tensors[n["f_bias"]]

    def cache_need(self):
        return None

    def state_need(self):
        s = self.spec
        return StateNeed((self.rt.ops.mlstm_state_size(s.num_heads, s.head_dim, s.v_head_dim),), "float32")

    def forward(self, x, batch, cache, state):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        hv = s.num_heads * s.v_head_dim
        proj = rt.linear(x, self.w_in)                    # float32 [n, q | k | v | gate | zi | zf]
        o_raw = rt.empty((n, hv), torch.float32)
        ops.mlstm_scan(proj, self.bias_i, self.bias_f, s.gate_cap, state, batch.q_start, batch.q_len, batch.slots, o_raw,
                       s.num_heads, s.head_dim, s.v_head_dim, few=batch.max_q_len <= 4)
        out = ops.mlstm_finish(o_raw, proj, 2 * s.num_heads * s.head_dim + hv, self.norm, s.norm_eps, rt.empty((n, hv), rt.act_dtype),
                               s.num_heads, s.v_head_dim)
        return rt.linear(out, self.w_o, slabs=True, defer=True)
