"""The plain implementation of the Rerizen decoder: whole sequences, no cache, no pages, no batching, one
function for each mechanism, NumPy float64.  It shares no code with `kipp_amd`; model folders are read with the
`safetensors` package.

Notation: a sequence has T tokens at positions 0 .. T-1; there are R copies X_1 .. X_R of the residual stream
("streams"), all equal to the embedding E[tokens] at the start.

    sublayer q of a layer     U = sum_r a_q[r] X_r;  Y = f_q(N_q(U));  X_t <- sum_r M_q[r, t] X_r + b_q[t] Y   (all t at once)
                              (f_1 the mixer, f_2 the feed-forward; without streams: X <- X + f_q(N_q(X)))
    norm                      N(x) = x / sqrt(mean(x^2) + eps) * w
    attention                 q = Wq x + bq, k = Wk x + bk, v = Wv x + bv; every head of q and k divided by its root mean
                              square; q(p) times 1 + c ln(floor((p + 1) / e) + 1); softmax_j<=i(scale q_h(i) . k_g(j)) v_g,
                              g = h // (H / G); a layer may read the keys and values of an earlier layer
    latent attention          cq = N(Wdq x), q = Wuq cq (a head is [unrotated | rotated]); Wdkv x = [c' | kr], c = N(c');
                              k_h = [Wuk_h c | rot(kr)], v_h = Wuv_h c; i sees j when 0 <= i - j < size;
                              o_h = softmax(scale q_h . k_h) v_h * sigmoid(Wg x)_h
    rotation                  pairs (2i, 2i + 1) turn by p * f_i, frequencies blended between f_i and f_i / factor by a
                              ramp over i, cosine and sine times 0.1 ln(factor) + 1
    matrix memory (mLSTM)     per head: li = cap tanh((Wi x + bi) / cap), lf = logsigmoid(cap tanh((Wf x + bf) / cap));
                              m_t = max(lf + m_(t-1), li); S_t = e^(lf + m_(t-1) - m_t) S_(t-1) + e^(li - m_t) k v^T,
                              n_t the same with k; o = S_t^T q / (max(|n_t . q|, e^(-m_t)) + 1e-6); o / rms(o) per head,
                              times the norm weight, times sigmoid(Wg x), then Wo
    feed-forward              Wd (silu(Wgate x) * (Wup x))
    output                    logits = H N_final(sum_r X_r) * logit_scale
"""
from __future__ import annotations

import json
import math
import os

import numpy as np

DTYPE = np.float64


def rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    x = np.asarray(x, dtype=DTYPE)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * np.asarray(w, dtype=DTYPE)


def linear(x, w, b=None):
    y = np.asarray(x, dtype=DTYPE) @ np.asarray(w, dtype=DTYPE).T
    return y if b is None else y + np.asarray(b, dtype=DTYPE)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def softmax_rows(scores, mask):
    """Softmax over the last axis of the entries that `mask` allows."""
    s = np.where(mask, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def causal(T):
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    return j <= i


def windowed(T, size):
    """i sees itself and the size - 1 positions before it."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def query_temperature(T, coef, every):
    p = np.arange(T)
    return 1.0 + coef * np.log(np.floor((p + 1) / every) + 1.0)


# ---- rotation ----------------------------------------------------------------------------------------------

def rotary_frequencies(dims, base, scaling=None):
    """f_i for i < dims / 2 and the factor on cosines and sines."""
    i = np.arange(dims // 2, dtype=DTYPE)
    f = base ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, magnitude):
    """x [T, ..., dims]: (x[2i], x[2i+1]) turned by positions * freqs[i]."""
    x = np.asarray(x, dtype=DTYPE)
    a = np.asarray(positions, dtype=DTYPE)[:, None] * freqs[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (freqs.shape[0],)
    c, s = (np.cos(a) * magnitude).reshape(shape), (np.sin(a) * magnitude).reshape(shape)
    u, v = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


# ---- mixers ------------------------------------------------------------------------------------------------

def attention_keys_values(h, w, m, eps, prefix):
    """What an attention layer keeps: its keys after the head norm, and its values."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms(linear(h, w[prefix + "k"], w[prefix + "k.b"]).reshape(T, G, d), eps)
    v = linear(h, w[prefix + "v"], w[prefix + "v.b"]).reshape(T, G, dv)
    return k, v


def attention(h, w, m, eps, prefix, kept=None):
    """Returns (mixer output, (keys, values)); with `kept` the keys and values of another layer are read."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(linear(h, w[prefix + "q"], w[prefix + "q.b"]).reshape(T, H, d), eps)
    if m.get("q_temp") is not None:
        q = q * query_temperature(T, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    k, v = kept if kept is not None else attention_keys_values(h, w, m, eps, prefix)
    out = np.zeros((T, H, dv), dtype=DTYPE)
    mask = causal(T)
    for head in range(H):
        g = head // (H // G)
        p = softmax_rows(q[:, head] @ k[:, g].T * m["scale"], mask)
        out[:, head] = p @ v[:, g]
    return linear(out.reshape(T, H * dv), w[prefix + "o"]), (k, v)


def latent_attention(h, w, m, eps, prefix):
    T = h.shape[0]
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = norm(linear(h, w[prefix + "dq"]), w[prefix + "dq.norm"], eps)
    q = linear(cq, w[prefix + "uq"]).reshape(T, H, d + dr)
    down = linear(h, w[prefix + "dkv"])
    c = norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    rot = m["rot"]
    freqs, magnitude = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    pos = np.arange(T)
    dims = rot["dims"]
    kr = down[:, rank:].copy()
    kr[:, :dims] = rotate_pairs(kr[:, :dims], pos, freqs, magnitude)
    qr = q[:, :, d:].copy()
    qr[:, :, :dims] = rotate_pairs(qr[:, :, :dims], pos, freqs, magnitude)
    k_plain = linear(c, w[prefix + "uk"]).reshape(T, H, d)
    v = linear(c, w[prefix + "uv"]).reshape(T, H, dv)
    gate = sigmoid(linear(h, w[prefix + "g"]))            # [T, H]
    size = (m.get("mask") or {}).get("size")
    mask = windowed(T, size) if size is not None else causal(T)
    out = np.zeros((T, H, dv), dtype=DTYPE)
    for head in range(H):
        s = (q[:, head, :d] @ k_plain[:, head].T + qr[:, head] @ kr.T) * m["scale"]
        out[:, head] = softmax_rows(s, mask) @ v[:, head] * gate[:, head:head + 1]
    return linear(out.reshape(T, H * dv), w[prefix + "o"])


def capped(z, cap):
    return cap * np.tanh(z / cap)


def mlstm(h, w, m, eps, prefix, state=None):
    """The matrix memory, token by token.  `state`: (S [H, d, dv], n [H, d], m [H]) to go on from; returns
    (mixer output, state)."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = linear(h, w[prefix + "q"]).reshape(T, H, d) * d ** -0.5
    k = linear(h, w[prefix + "k"]).reshape(T, H, d)
    v = linear(h, w[prefix + "v"]).reshape(T, H, dv)
    li = capped(linear(h, w[prefix + "i"], w[prefix + "i.b"]), cap)
    lf = log_sigmoid(capped(linear(h, w[prefix + "f"], w[prefix + "f.b"]), cap))
    if state is None:
        state = (np.zeros((H, d, dv), dtype=DTYPE), np.zeros((H, d), dtype=DTYPE), np.zeros(H, dtype=DTYPE))
    S, n, mx = (np.array(a, dtype=DTYPE) for a in state)
    out = np.zeros((T, H, dv), dtype=DTYPE)
    for t in range(T):
        m_new = np.maximum(lf[t] + mx, li[t])
        keep, take = np.exp(lf[t] + mx - m_new), np.exp(li[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = m_new
        num = np.einsum("hdv,hd->hv", S, q[t])
        den = np.maximum(np.abs(np.einsum("hd,hd->h", n, q[t])), np.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    o = rms(out, eps).reshape(T, H * dv) * np.asarray(w[prefix + "norm"], dtype=DTYPE)
    o = o * sigmoid(linear(h, w[prefix + "g"]))
    return linear(o, w[prefix + "o"]), (S, n, mx)


def feed_forward(h, w, prefix):
    g = linear(h, w[prefix + "gate"])
    return linear(g * sigmoid(g) * linear(h, w[prefix + "up"]), w[prefix + "down"])


# ---- the streams --------------------------------------------------------------------------------------------

def streams_read(X, a):
    """U = sum_r a[r] X_r for X [R, T, width]."""
    return np.tensordot(np.asarray(a, dtype=DTYPE), X, axes=(0, 0))


def streams_write(X, M, b, Y):
    """X_t <- sum_r M[r, t] X_r + b[t] Y, all t from the old X."""
    M, b = np.asarray(M, dtype=DTYPE), np.asarray(b, dtype=DTYPE)
    return np.einsum("rt,rnw->tnw", M, X) + b[:, None, None] * Y[None]


# ---- the model ----------------------------------------------------------------------------------------------

def forward(config, w, tokens, layers_out=None):
    """Logits [T, vocab] of a whole sequence.  `layers_out`: a list that receives the residual stream (the sum
    of the streams) after every layer."""
    eps = config["norm"]["eps"]
    R = config.get("streams")
    x = np.asarray(w["embed"], dtype=DTYPE)[np.asarray(tokens, dtype=np.int64)]
    X = np.stack([x] * R) if R is not None else x
    kept = {}
    for i, layer in enumerate(config["layers"]):
        m, name = layer["mixer"], f"l{i}."
        subs = [(1, "mix.")] + ([(2, "mlp.")] if layer.get("mlp") is not None else [])
        for q, prefix in subs:
            u = streams_read(X, w[f"{name}hc{q}.in"]) if R is not None else X
            h = norm(u, w[f"{name}norm{q}"], eps)
            if q == 2:
                y = feed_forward(h, w, name + prefix)
            elif layer["type"] == "attention":
                y, kv = attention(h, w, m, eps, name + prefix, kept.get(m.get("kv_from")) if m.get("kv_from") is not None else None)
                if m.get("kv_from") is None:
                    kept[i] = kv
            elif layer["type"] == "latent_attention":
                y = latent_attention(h, w, m, eps, name + prefix)
            elif layer["type"] == "mlstm":
                y, _ = mlstm(h, w, m, eps, name + prefix)
            else:
                raise ValueError(layer["type"])
            X = streams_write(X, w[f"{name}hc{q}.mix"], w[f"{name}hc{q}.out"], y) if R is not None else X + y
        if layers_out is not None:
            layers_out.append(X.sum(axis=0) if R is not None else X.copy())
    x = X.sum(axis=0) if R is not None else X
    return linear(norm(x, w["final.norm"], eps), w["head"]) * config.get("logit_scale", 1.0)


def load_folder(model_dir):
    """(config dict, {name: float64 array}) of a model folder."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    w = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(torch.float64).numpy()
    return config, w
