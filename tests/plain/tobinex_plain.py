"""The plain implementation of the Tobinex decoder: whole sequences, no cache,
no pages, no batching, one function for each mechanism, NumPy float64.  It
shares no code with `kipp_amd`; model folders are read with the `safetensors`
package.

Notation: a sequence has T tokens at positions 0 .. T-1; a layer maps the
residual stream X [T, width] to the next one.

    embedding      X = E[tokens] * s
    layer          X <- N1(a X + mixer(X));  X <- N2(a X + ff(X))     (norm after the sum; a = postln_alpha)
    norm           N(x) = x / sqrt(mean(x^2) + eps) * (1 + w)
    attention      q = Wq x, k = Wk x, v = Wv x; q and k each normed over the WHOLE projection (all heads at
                   once, plain weight); score_h(i, j) = scale * q_h(i) . k_c(j) - r1_h * ln(1 + r2_h * (i - j)),
                   c = h // (H / G); i sees j when j <= i and (i - j < size or j < keep_first);
                   p_h(i, j) = exp(score_h(i, j)) / (exp(sink_h) + sum_j' exp(score_h(i, j')));
                   p'_h = sum_g T[h, g] p_g;  o_h(i) = sum_j p'_h(i, j) v_c(j);
                   y = Wo (concat_h o_h * sigmoid(Wg x))
    feed-forward   Wd (silu(Wgate x) * (Wup x))
    output         logits = E N_final(X)        (the table without its scale)
"""
from __future__ import annotations

import json
import os

import numpy as np

DTYPE = np.float64


def rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    x = np.asarray(x, dtype=DTYPE)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def one_plus_norm(x, w, eps):
    """The layer norms: the tensor holds the offset of the weight from one."""
    return rms(x, eps) * (1.0 + np.asarray(w, dtype=DTYPE))


def plain_weight_norm(x, w, eps):
    """The query/key norm: over the whole projection, plain weight."""
    return rms(x, eps) * np.asarray(w, dtype=DTYPE)


def embed(table, tokens, scale):
    return np.asarray(table, dtype=DTYPE)[np.asarray(tokens, dtype=np.int64)] * scale


def linear(x, w):
    return np.asarray(x, dtype=DTYPE) @ np.asarray(w, dtype=DTYPE).T


def visible(T, size, keep_first):
    """mask[i, j]: position i sees position j.  `size` None: every earlier key."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    near = (i - j < size) if size is not None else np.ones((T, T), dtype=bool)
    return (j <= i) & (near | (j < keep_first))


def distance_bias(T, r1, r2):
    """[H, T, T]: r1_h * ln(1 + r2_h * (i - j)) for j <= i (0 elsewhere; those are masked anyway)."""
    dist = np.maximum(np.arange(T)[:, None] - np.arange(T)[None, :], 0).astype(DTYPE)
    r1 = np.asarray(r1, dtype=DTYPE)[:, None, None]
    r2 = np.asarray(r2, dtype=DTYPE)[:, None, None]
    return r1 * np.log1p(r2 * dist[None])


def sink_softmax(scores, mask, sink):
    """[H, T, T] -> weights whose denominator also holds exp(sink_h), once."""
    sink = np.asarray(sink, dtype=DTYPE)[:, None, None]
    s = np.where(mask[None], scores, -np.inf)
    top = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.exp(s - top)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(sink - top))


def mix_heads(p, talk):
    """p'[h] = sum_g talk[h, g] p[g]."""
    return np.einsum("hg,gij->hij", np.asarray(talk, dtype=DTYPE), p)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def attention(x, w, m, eps):
    """`w`: the mixer's tensors by local name; `m`: its sizes and constants."""
    T = x.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    mask_cfg = m.get("mask") or {}
    q = plain_weight_norm(linear(x, w["q"]), w["q.norm"], eps).reshape(T, H, d)
    k = plain_weight_norm(linear(x, w["k"]), w["k.norm"], eps).reshape(T, G, d)
    v = linear(x, w["v"]).reshape(T, G, dv)
    kv_of = np.arange(H) // (H // G)
    scores = np.einsum("ihd,jhd->hij", q, k[:, kv_of]) * m["scale"] - distance_bias(T, w["r1"], w["r2"])
    p = sink_softmax(scores, visible(T, mask_cfg.get("size"), mask_cfg.get("keep_first", 0) or 0), w["sink"])
    p = mix_heads(p, w["talk"])
    o = np.einsum("hij,jhe->ihe", p, v[:, kv_of]).reshape(T, H * dv)
    return linear(o * sigmoid(linear(x, w["g"])), w["o"])


def dense_ff(x, w):
    g = linear(x, w["gate"])
    return linear(g * sigmoid(g) * linear(x, w["up"]), w["down"])


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward_whole(cfg, weights, tokens, layers_out=None):
    """float64 logits [T, vocab] of one whole sequence.  `layers_out`: a list that receives the residual
    stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = embed(weights["embed"], tokens, cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(f"layer type {layer['type']!r}")
        x = one_plus_norm(alpha * x + attention(x, sub(weights, p + "mix."), layer["mixer"], eps), weights[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = one_plus_norm(alpha * x + dense_ff(x, sub(weights, p + "mlp.")), weights[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    x = one_plus_norm(x, weights["final.norm"], eps)
    return linear(x, weights["embed"])


def load_folder(folder):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as f:
        cfg = json.load(f)
    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).float().numpy().astype(DTYPE)
    return cfg, weights
