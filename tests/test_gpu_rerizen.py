"""The Rerizen design on the GPU against its plain implementation: every new kernel alone (crafted inputs at the edges),
then the engine under every cutting in both precisions, tight pools, slots used again, long decoding, recorded steps,
other sizes, generation through the scheduler, the trace replay and the command line."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers as H
from tests.plain import rerizen_plain as P

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHAPES = ("rerizen-tiny-a", "rerizen-tiny-b")
LENGTHS = [1, 19, 45, 80, 131]
TOL = {"float32": 1e-9, "bfloat16": 3e-3}     # float32 is the sharp test; narrow widths make bfloat16 rows noisy


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("rerizen")
    return {(shape, dtype): write_random_model(str(root / f"{shape}-{dtype}"), shape_config(shape), seed=60 + i, dtype=dtype)
            for i, shape in enumerate(SHAPES) for dtype in ("float32", "bfloat16")}


_plain_cache = {}


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        cfg, w = P.load_folder(folder)
        _plain_cache[key] = P.forward(cfg, w, list(tokens))
    return _plain_cache[key]


def close(got, ref, tol, what):
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    worst = max(float(np.sum((g - r) ** 2) / np.sum(r ** 2)) for g, r in zip(got.astype(np.float64), ref))
    assert worst <= tol, f"{what}: NMSE {worst:.3e} exceeds {tol:.1e}"


def engine_of(folder, dtype, page=16, **kw):
    from kipp_amd.engine import Engine
    kw.setdefault("max_tokens", 1024)
    return Engine.from_folder(folder, dtype=dtype, page_size=page, share_prefixes=False, **kw)


def dev(a, ty=None):
    import torch
    return None if a is None else torch.tensor(np.asarray(a), device="cuda:0", dtype=ty)


def bf16(x):
    import torch
    return torch.tensor(np.asarray(x, dtype=np.float32)).bfloat16().float().numpy().astype(np.float64)


# =============================================================================== the kernels alone

@pytest.mark.parametrize("R, width", [(1, 40), (2, 192), (3, 1000), (8, 2304)])
def test_streams_kernels(R, width):
    import torch
    from kipp_amd.csrc import ops
    rng = np.random.default_rng(R)
    n = 5
    table = rng.normal(size=(9, width)).astype(np.float32)
    toks = [3, 0, 8, 8, 1]
    X = ops.streams_open(dev(table), dev(toks, torch.int32), torch.empty((n, R, width), device="cuda:0"))
    assert all(np.array_equal(X.cpu().numpy()[:, r], table[toks]) for r in range(R))
    x0 = rng.normal(size=(n, R, width)).astype(np.float32)
    delta = rng.normal(size=(3, n, width)).astype(np.float32)
    mix, outw, inw = (rng.normal(size=s).astype(np.float32) for s in ((R, R), (R,), (R,)))
    w = rng.normal(size=width).astype(np.float32)
    ref_x = P.streams_write(x0.transpose(1, 0, 2).astype(np.float64), mix, outw, delta.astype(np.float64).sum(0))
    ref_h = P.norm(P.streams_read(ref_x, inw), w, 1e-5)
    X = dev(x0)
    h = ops.streams_step(X, dev(delta), dev(mix), dev(outw), dev(inw), dev(w), 1e-5, torch.empty((n, width), device="cuda:0"))
    assert np.allclose(X.cpu().numpy().transpose(1, 0, 2), ref_x, rtol=2e-5, atol=2e-5)
    assert np.allclose(h.cpu().numpy(), ref_h, rtol=3e-5, atol=3e-5)
    # the read alone, into bfloat16; the write alone; the closing sum of named rows
    hb = ops.streams_step(X, None, None, None, dev(inw), dev(w), 1e-5, torch.empty((n, width), device="cuda:0", dtype=torch.bfloat16))
    assert np.allclose(hb.float().cpu().numpy(), ref_h, rtol=1e-2, atol=1e-2)
    X2 = dev(x0)
    ops.streams_step(X2, dev(delta[0]), dev(mix), dev(outw), None, None, 0.0, None)
    assert np.allclose(X2.cpu().numpy().transpose(1, 0, 2), P.streams_write(x0.transpose(1, 0, 2).astype(np.float64), mix, outw, delta[0].astype(np.float64)),
                       rtol=2e-5, atol=2e-5)
    which = [4, 1]
    s = ops.streams_close(dev(x0), dev(delta), dev(mix), dev(outw), dev(which, torch.int32), torch.empty((2, width), device="cuda:0"))
    assert np.allclose(s.cpu().numpy(), ref_x.sum(0)[which], rtol=3e-5, atol=3e-5)
    # the last read of a forward pass: named rows, the write carried out but not stored, the sum of the copies normed
    X3 = dev(x0)
    h3 = ops.streams_step(X3, dev(delta), dev(mix), dev(outw), dev(np.ones(R, np.float32)), dev(w), 1e-5,
                          torch.empty((2, width), device="cuda:0"), which=dev(which, torch.int32), store=False)
    assert np.allclose(h3.cpu().numpy(), P.norm(ref_x.sum(0)[which], w, 1e-5), rtol=3e-5, atol=3e-5) and np.array_equal(X3.cpu().numpy(), x0)
    s = ops.streams_close(dev(x0), None, None, None, None, torch.empty((n, width), device="cuda:0"))
    assert np.allclose(s.cpu().numpy(), x0.astype(np.float64).sum(1), rtol=1e-5, atol=1e-5)


class PagedCase:
    """T tokens of one sequence in pages handed out in a scrambled order; `queries` None: one prompt portion of all T rows,
    else each listed position as a single token of an entry of its own that shares the pages."""

    def __init__(self, T, page, queries=None, seed=0):
        import torch
        self.T, self.page = T, page
        blocks = -(-T // page)
        rng = np.random.default_rng(seed)
        self.pages = blocks + 3
        order = rng.permutation(self.pages)[:blocks]
        if queries is None:
            self.rows, pos, seq, tables = T, list(range(T)), [0] * T, [list(order)]
        else:
            self.rows, pos, seq, tables = len(queries), list(queries), list(range(len(queries))), [list(order)] * len(queries)
        self.positions, self.seq_of = dev(pos, torch.int32), dev(seq, torch.int32)
        self.table = dev(tables, torch.int32)
        self.pos = pos


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H_, G, d, dv, norm, temp", [(4, 2, 32, 32, "plain", (0.5, 8)), (6, 3, 24, 40, "plain", None), (3, 1, 80, 16, "weighted", (1.5, 3)),
                                                      (5, 5, 16, 200, "none", (0.2, 1))])
def test_head_prepare_and_wide_attention(dtype, H_, G, d, dv, norm, temp):
    """Biases, the head norm in its three modes, the query factor, the cache write and the generic attention with values
    of their own width, for a prompt portion from slabs and for single tokens anywhere."""
    import torch
    from kipp_amd.csrc import ops
    rng = np.random.default_rng(H_)
    T, page, scale, eps = 70, 16, 0.21, 1e-5
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    width = H_ * d + G * d + G * dv
    proj = rng.normal(size=(2, T, width + 5)).astype(np.float32)
    bias = rng.normal(size=width).astype(np.float32)
    qw, kw = (1 + 0.2 * rng.normal(size=d)).astype(np.float32), (1 + 0.2 * rng.normal(size=d)).astype(np.float32)
    x = proj.astype(np.float64).sum(0)[:, :width] + bias
    q, k, v = x[:, :H_ * d].reshape(T, H_, d), x[:, H_ * d:H_ * d + G * d].reshape(T, G, d), x[:, H_ * d + G * d:].reshape(T, G, dv)
    if norm != "none":
        q, k = P.rms(q, eps), P.rms(k, eps)
    if norm == "weighted":
        q, k = q * qw, k * kw
    if temp is not None:
        q = q * P.query_temperature(T, *temp)[:, None, None]
    if dtype == "bfloat16":
        q, k, v = bf16(q), bf16(k), bf16(v)
    ref = np.zeros((T, H_, dv))
    for h in range(H_):
        p = P.softmax_rows(q[:, h] @ k[:, h // (H_ // G)].T * scale, P.causal(T))
        ref[:, h] = p @ v[:, h // (H_ // G)]
    for queries in (None, [69, 0, 16, 33]):
        case = PagedCase(T, page, queries, seed=d)
        kc = torch.zeros((case.pages, G, page, d), dtype=act, device="cuda:0")
        vc = torch.zeros((case.pages, G, page, dv), dtype=act, device="cuda:0")
        whole = PagedCase(T, page, None, seed=d)       # the same page order: fills the pages
        args = (H_, G, d, dv, dev(bias), norm, eps, dev(qw), dev(kw)) + (temp if temp is not None else (0.0, 0))
        qd = ops.head_prepare(dev(proj), torch.empty((T, H_ * d), dtype=act, device="cuda:0"), kc, vc, whole.positions, whole.seq_of,
                              whole.table, *args)
        if queries is not None:
            qd = qd[queries].contiguous()
        out = ops.paged_attention_wide(qd, kc, vc, torch.empty((case.rows, H_ * dv), dtype=act, device="cuda:0"), case.positions,
                                       case.seq_of, case.table, H_, G, d, dv, scale)
        want = ref.reshape(T, H_ * dv)[case.pos]
        tol = 2e-5 if dtype == "float32" else 2e-2
        assert np.allclose(out.float().cpu().numpy(), want, rtol=tol, atol=tol * np.abs(want).max()), (dtype, queries)


def attention_batch(case, T, queries):
    """What `paged_attention` reads of a step's batch, for one prompt portion of T rows or for single tokens at `queries`."""
    import types

    import torch
    from kipp_amd.engine.batch import StepBatch

    class B:
        pass
    b = B()
    b.n_portions, b.n_decode = (1, 0) if queries is None else (0, len(queries))
    b.q_start = dev([0] if queries is None else list(range(len(queries))), torch.int32)
    b.q_len = dev([T] if queries is None else [1] * len(queries), torch.int32)
    b.positions, b.seq_of_token = case.positions, case.seq_of
    b.decode_rows = dev(list(range(len(queries))) if queries else [0], torch.int32)
    b.max_decode_ctx = T
    b.n_tokens = case.rows
    b.host = {"q_start": [0] if queries is None else list(range(len(queries))), "q_len": [T] if queries is None else [1] * len(queries),
              "ctx_len": [T] if queries is None else [p_ + 1 for p_ in queries]}
    b.step_cache = {}
    b.upload = types.MethodType(StepBatch.upload, b)
    b.tokens = case.positions
    return b


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", [0, 2, 15, 16, 255, 256])
def test_a_far_key_takes_the_softmax(dtype, key):
    """One key among 300, at the sequence's start and on both sides of page and tile borders, points where the last query
    points after the head norm and the query factor: the last row's result is that key's value, for the row of a prompt
    portion and for a single token, on the matrix-core kernels and on the generic one."""
    import torch
    from kipp_amd.csrc import ops
    from kipp_amd.parts.mixer import paged_attention
    from kipp_amd.runtime import Runtime
    rt = Runtime(dtype)
    act = rt.act_dtype
    H_, G, d, dv, T, page, scale = 4, 2, 32, 32, 300, 16, 1.0
    rng = np.random.default_rng(key)
    proj = rng.normal(size=(T, H_ * d + G * d + G * dv)).astype(np.float32)
    u = rng.normal(size=d).astype(np.float32)
    for h in range(H_):
        proj[T - 1, h * d:(h + 1) * d] = 5.0 * u             # the norm takes the length away, the direction stays
    for g in range(G):
        proj[key, H_ * d + g * d:H_ * d + (g + 1) * d] = -3.0 * u if key == T - 1 else 3.0 * u
        proj[key, H_ * d + G * d + g * dv:H_ * d + G * d + (g + 1) * dv] = 200.0
    for fast in ([False, True] if dtype == "bfloat16" else [False]):
        for queries in (None, [T - 1]):
            whole, case = PagedCase(T, page, None, seed=1), PagedCase(T, page, queries, seed=1)
            kc = torch.zeros((case.pages, G, page, d), dtype=act, device="cuda:0")
            vc = torch.zeros((case.pages, G, page, dv), dtype=act, device="cuda:0")
            q = ops.head_prepare(dev(proj), torch.empty((T, H_ * d), dtype=act, device="cuda:0"), kc, vc, whole.positions, whole.seq_of,
                                 whole.table, H_, G, d, dv, None, "plain", 1e-5, None, None, 0.5, 64)
            if queries is not None:
                q = q[queries].contiguous()
            out = torch.zeros((case.rows, H_ * dv), dtype=act, device="cuda:0")
            paged_attention(rt, attention_batch(case, T, queries), q, out, kc, vc, page, case.table, H_, G, d, dv, scale, None, fast)
            last = out[-1].float().cpu().numpy()
            assert np.allclose(last, 200.0, rtol=2e-2), (dtype, fast, queries, last[:4])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, d, dr, dv, q_rank, rank, rot_dims, window, fast", [
    (4, 32, 16, 24, 64, 48, 16, 40, True), (5, 24, 8, 20, 40, 36, 8, None, False), (2, 16, 12, 48, 24, 20, 8, 7, False),
    (16, 64, 32, 64, 96, 224, 32, 100, True), (3, 8, 6, 8, 8, 298, 6, 1, False), (20, 16, 16, 16, 32, 48, 16, 33, False)])
def test_latent_kernels_with_a_key_that_stands_out(dtype, heads, d, dr, dv, q_rank, rank, rot_dims, window, fast):
    """prepare, absorb, attention over the cached rows (the matrix-core kernels where they take the sizes, else the generic
    one reading values out of the key rows) and expand, against the plain mixer's steps; then one latent made to stand out,
    placed just inside and just outside the window, in a prompt row and for a single token."""
    import torch
    from kipp_amd.csrc import ops
    from kipp_amd.parts.mixer import paged_attention
    from kipp_amd.runtime import Runtime
    rt = Runtime(dtype)
    act = rt.act_dtype
    rng = np.random.default_rng(heads * 7 + d)
    T, page, scale, eps = 150, 16, 0.11, 1e-5
    row = rank + dr
    m = {"heads": heads, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": q_rank, "kv_rank": rank, "scale": scale,
         "rot": {"base": 777.0, "dims": rot_dims, "scaling": {"factor": 5.0, "original": 40, "fast": 10.0, "slow": 1.0}},
         "mask": {"size": window} if window else None}
    freqs, mag = P.rotary_frequencies(rot_dims, 777.0, m["rot"]["scaling"])
    w = {"uq": rng.normal(size=(heads * (d + dr), q_rank)) / math.sqrt(q_rank), "uk": rng.normal(size=(heads * d, rank)) / math.sqrt(rank),
         "uv": rng.normal(size=(heads * dv, rank)) / math.sqrt(rank), "dq.norm": 1 + 0.1 * rng.normal(size=q_rank),
         "dkv.norm": 1 + 0.1 * rng.normal(size=rank)}
    rnd = (lambda a: bf16(a)) if dtype == "bfloat16" else (lambda a: np.asarray(a, dtype=np.float64))
    w = {k_: rnd(v_) for k_, v_ in w.items()}
    for far in (None, "in", "out"):
        proj = rng.normal(size=(T, q_rank + row + heads)).astype(np.float32)
        last = T - 1
        if far is not None and window is not None and 1 < window < T:
            key = last - window + 1 if far == "in" else last - window
            special = key
        else:
            special = None
        x = proj.astype(np.float64)
        cq = rnd(P.norm(x[:, :q_rank], w["dq.norm"], eps))
        c = P.norm(x[:, q_rank:q_rank + rank], w["dkv.norm"], eps)
        kr = x[:, q_rank + rank:q_rank + row].copy()
        kr[:, :rot_dims] = P.rotate_pairs(kr[:, :rot_dims], np.arange(T), freqs, mag)
        q = (cq @ w["uq"].T).reshape(T, heads, d + dr)
        if special is not None:
            # every head's last query points along the latent of `special`, far longer than any other score
            target = rnd(c[special])
            for h in range(heads):
                uk = w["uk"][h * d:(h + 1) * d]
                q[last, h, :d] = 400.0 * (uk @ target) / max(np.linalg.norm(uk @ target), 1e-9)
        rows_cache = rnd(np.concatenate([c, kr], axis=1))
        qr = q[:, :, d:].copy()
        qr[:, :, :rot_dims] = P.rotate_pairs(qr[:, :, :rot_dims], np.arange(T), freqs, mag)
        mask = P.windowed(T, window) if window else P.causal(T)
        gate = P.sigmoid(x[:, q_rank + row:])
        ref = np.zeros((T, heads, dv))
        for h in range(heads):
            ql = rnd(np.concatenate([q[:, h, :d] @ w["uk"][h * d:(h + 1) * d], qr[:, h]], axis=1))
            p = P.softmax_rows(ql @ rows_cache.T * scale, mask)
            ref[:, h] = (p @ rows_cache[:, :rank]) @ w["uv"][h * dv:(h + 1) * dv].T * gate[:, h:h + 1]
        ref = ref.reshape(T, heads * dv)
        for queries in (None, [last, 0, 17]):
            whole, case = PagedCase(T, page, None, seed=3), PagedCase(T, page, queries, seed=3)
            cache = torch.zeros((case.pages, 1, page, row), dtype=act, device="cuda:0")
            freq_d = dev(freqs.astype(np.float32))
            cqd = ops.latent_prepare(dev(proj), torch.empty((T, q_rank), dtype=act, device="cuda:0"), cache, whole.positions, whole.seq_of,
                                     whole.table, q_rank, rank, dr, dev(w["dq.norm"].astype(np.float32)), dev(w["dkv.norm"].astype(np.float32)),
                                     eps, freq_d, rot_dims, mag)
            assert np.allclose(cqd.float().cpu().numpy(), cq, rtol=1e-2 if dtype == "bfloat16" else 1e-5, atol=1e-5)
            qd = dev(q.astype(np.float32))                       # the product W_uq cq, as float32 rows
            ql = ops.latent_absorb(qd.view(T, -1), dev(w["uk"].astype(np.float32)).to(act), torch.empty((T, heads * row), dtype=act, device="cuda:0"),
                                   whole.positions, freq_d, rot_dims, mag, heads, d, dr, rank)
            if queries is not None:
                ql = ql[queries].contiguous()
            use_fast = fast and dtype == "bfloat16"
            widthv = row if use_fast else rank
            lat = torch.zeros((case.rows, heads * widthv), dtype=act, device="cuda:0")

            b = attention_batch(case, T, queries)
            paged_attention(rt, b, ql, lat, cache, cache, page, case.table, heads, 1, row, widthv, scale, window, use_fast)
            uv_t = dev(w["uv"].astype(np.float32)).to(act).view(heads, dv, rank).transpose(1, 2).contiguous()
            gate_src = dev(proj) if queries is None else dev(proj[queries])
            out = ops.latent_expand(lat, uv_t, torch.empty((case.rows, heads * dv), dtype=act, device="cuda:0"), heads, rank, dv,
                                    gate=gate_src, gate_at=q_rank + row)
            want = ref[case.pos]
            tol = 3e-4 if dtype == "float32" else 3e-2
            err = np.abs(out.float().cpu().numpy() - want).max() / np.abs(want).max()
            assert err < tol, (dtype, far, queries, err)


@pytest.mark.parametrize("heads, d, dv", [(4, 32, 32), (3, 20, 72), (2, 36, 16), (1, 128, 130), (2, 300, 24), (5, 3, 1)])
def test_mlstm_scan_and_finish(heads, d, dv):
    """The recurrence over portions of several entries at once, from states left by earlier launches, in slots in any
    order, against the plain mixer; gates driven to both ends of their cap."""
    import torch
    from kipp_amd.csrc import ops
    rng = np.random.default_rng(d)
    width, cap, eps = 24, 5.0, 1e-5
    m = {"heads": heads, "dim": d, "vdim": dv, "gate_cap": cap}
    w = {"q": rng.normal(size=(heads * d, width)) / 3, "k": rng.normal(size=(heads * d, width)) / 3, "v": rng.normal(size=(heads * dv, width)),
         "g": rng.normal(size=(heads * dv, width)), "o": np.eye(heads * dv), "norm": 1 + 0.2 * rng.normal(size=heads * dv),
         "i": 3 * rng.normal(size=(heads, width)), "i.b": rng.normal(size=heads), "f": 3 * rng.normal(size=(heads, width)), "f.b": 2 + rng.normal(size=heads)}
    lengths = {"a": [5, 1, 1, 30], "b": [64, 2], "c": [1, 1, 1, 1]}
    hs = {r: rng.normal(size=(sum(n), width)) for r, n in lengths.items()}
    ref = {r: P.mlstm(hs[r], w, m, eps, "")[0] for r in hs}
    size = ops.mlstm_state_size(heads, d, dv)
    state = torch.zeros((6, size + 3), device="cuda:0")
    slot = {"a": 4, "b": 0, "c": 2}
    fed = {r: 0 for r in hs}
    got = {r: [] for r in hs}
    w_in = np.concatenate([w[k_] for k_ in ("q", "k", "v", "g", "i", "f")])
    for step in range(4):
        live = [r for r in hs if step < len(lengths[r])]
        counts = [lengths[r][step] for r in live]
        rows = np.concatenate([hs[r][fed[r]:fed[r] + n] for r, n in zip(live, counts)])
        proj = dev((rows @ w_in.T).astype(np.float32))
        starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
        o_raw = torch.empty((rows.shape[0], heads * dv), device="cuda:0")
        ops.mlstm_scan(proj, dev(w["i.b"].astype(np.float32)), dev(w["f.b"].astype(np.float32)), cap, state, dev(starts, torch.int32),
                       dev(counts, torch.int32), dev([slot[r] for r in live], torch.int32), o_raw, heads, d, dv)
        out = ops.mlstm_finish(o_raw, proj, 2 * heads * d + heads * dv, dev(w["norm"].astype(np.float32)), eps,
                               torch.empty((rows.shape[0], heads * dv), device="cuda:0"), heads, dv).cpu().numpy()
        for r, n, s in zip(live, counts, starts):
            got[r].append(out[s:s + n])
            fed[r] += n
    for r in hs:
        g = np.concatenate(got[r])
        assert np.allclose(g, ref[r], rtol=2e-3, atol=2e-3 * np.abs(ref[r]).max()), (r, np.abs(g - ref[r]).max())
    assert (state[[1, 3, 5]] == 0).all() and (state[:, size:] == 0).all()      # nothing outside the entries' slots


@pytest.mark.parametrize("heads, d, dv", [(3, 128, 80), (2, 200, 40), (2, 256, 72), (2, 24, 70)])
def test_mlstm_scan_for_few_tokens_gives_the_same_bits(heads, d, dv):
    """Single tokens take a build with fewer, larger workgroups: the same state and the same output, bit for bit."""
    import torch
    from kipp_amd.csrc import ops
    rng = np.random.default_rng(4)
    size = ops.mlstm_state_size(heads, d, dv)
    proj = dev(rng.normal(size=(6, 2 * heads * d + 2 * heads * dv + 2 * heads)).astype(np.float32))
    start = torch.tensor(rng.normal(size=(4, size)).astype(np.float32), device="cuda:0")
    copies = -(-dv // ops.mlstm_columns(d))
    n0 = start[:, heads * d * dv:heads * d * dv + heads * d].clone()
    for c in range(copies):         # the copies of n and m of a slot hold the same numbers
        start[:, heads * d * dv + c * heads * d:heads * d * dv + (c + 1) * heads * d] = n0
        start[:, heads * d * dv + copies * heads * d + c * heads:heads * d * dv + copies * heads * d + (c + 1) * heads] = start[:, -heads - 4:-4].abs()
    outs = []
    for few in (False, True):
        state = start.clone()
        o = torch.empty((6, heads * dv), device="cuda:0")
        for step in range(2):
            rows = proj[3 * step:3 * step + 3].contiguous()
            ops.mlstm_scan(rows, dev(np.zeros(heads, np.float32)), dev(np.ones(heads, np.float32)), 7.0, state, dev([0, 1, 2], torch.int32),
                           dev([1, 1, 1], torch.int32), dev([2, 0, 3], torch.int32), o[3 * step:3 * step + 3], heads, d, dv, few=few)
        outs.append((o.cpu().numpy(), state.cpu().numpy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


# =============================================================================== the engine

def requests_of(vocab, seed=0, lengths=LENGTHS):
    return {f"r{i}": H.random_tokens(seed * 100 + i, n, vocab) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype, page", [("float32", 16), ("bfloat16", 16), ("bfloat16", 32), ("bfloat16", 8)])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuttings_match_plain(folders, shape, dtype, page, cut):
    """Whole prompts, the last tokens one by one, portions of changing size down to two tokens, and mixed batches in a
    pool that only holds the live requests and has four state slots (pages and slots are used again)."""
    folder = folders[(shape, dtype)]
    vocab = P.load_folder(folder)[0]["vocab"]
    requests = requests_of(vocab)
    if cut == "mixed":
        requests.update({f"s{i}": H.random_tokens(900 + i, n, vocab) for i, n in enumerate(LENGTHS)})
        steps = H.mixed(requests, seed=5)
        engine = engine_of(folder, dtype, page, max_tokens=None, num_pages=H.peak_pages(requests, steps, page), max_requests=4)
    else:
        engine = engine_of(folder, dtype, page)
        steps = {"whole": H.whole, "tail": H.tail_one_by_one, "portions": H.changing_portions}[cut](requests)
    got = H.replay(engine, requests, steps)
    for rid, toks in requests.items():
        close(got[rid], plain_logits(folder, toks), TOL[dtype], f"{shape}/{dtype}/{page}/{cut}/{rid}")
    assert engine.cache.free_pages() == [g.pool.num_pages for g in engine.cache.groups]
    if dtype == "bfloat16" and page == 16:
        # the first shape's attention runs on the matrix cores throughout, the second's sizes leave them
        assert (engine.rt.generic_attention_launches > 0) == (shape == "rerizen-tiny-b")


@pytest.mark.parametrize("shape", SHAPES)
def test_float32_cuttings_are_bitwise_equal(folders, shape):
    """In float32 every sum runs in an order that the token's own position fixes: how the prompt was cut, what else was
    in the batch and which pages and slots were used change no bit."""
    folder = folders[(shape, "float32")]
    requests = requests_of(P.load_folder(folder)[0]["vocab"], seed=3)
    base = H.replay(engine_of(folder, "float32"), requests, H.whole(requests))
    for maker in (H.tail_one_by_one, H.changing_portions, lambda r: H.mixed(r, seed=11)):
        steps = maker(requests)
        order = list(np.random.default_rng(1).permutation(64))
        got = H.replay(engine_of(folder, "float32", page_order=order, max_requests=5), requests, steps)
        for rid in requests:
            assert np.array_equal(got[rid], base[rid]), f"{shape}/{rid}: bits differ between cuttings"


def _one_layer(kind, mixer, **top):
    cfg = {"architecture": "Rerizen", "vocab": 90, "width": 64, "streams": 2, "norm": {"eps": 1e-5}, "logit_scale": 2.0,
           "layers": [{"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": 48}}]}
    cfg.update(top)
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_a_small_pool_and_one_slot(tmp_path, dtype):
    """A window of 20 in pages of 16 over an mLSTM layer: 200 tokens pass through four pages and the one state slot, which
    a second request then takes over (its state must start at zero, not where the first left it)."""
    from kipp_amd.weights import write_random_model
    cfg = _one_layer("latent_attention", {"heads": 4, "dim": 16, "rot_dim": 16, "vdim": 16, "q_rank": 32, "kv_rank": 48, "scale": 0.2,
                                          "rot": {"base": 1000.0, "dims": 16}, "mask": {"size": 20}})
    cfg["layers"].append({"type": "mlstm", "mixer": {"heads": 2, "dim": 16, "vdim": 24, "gate_cap": 8.0}, "mlp": None})
    folder = write_random_model(str(tmp_path / "two"), cfg, seed=8, dtype=dtype)
    tokens = {"r": H.random_tokens(77, 200, 90), "next": H.random_tokens(78, 40, 90)}
    engine = engine_of(folder, dtype, 16, max_tokens=None, num_pages=4, max_requests=1)
    steps = [([("r", 10)], [])] + [([("r", 1)], []) for _ in range(60)] + [([("r", 7)], []), ([("r", 2)], [])] \
        + [([("r", 1)], []) for _ in range(121)]
    steps[-1] = (steps[-1][0], ["r"])
    steps += [([("next", 33)], [])] + [([("next", 1)], []) for _ in range(7)]
    steps[-1] = (steps[-1][0], ["next"])
    got = H.replay(engine, tokens, steps)
    for rid in tokens:
        close(got[rid], plain_logits(folder, tokens[rid]), TOL[dtype], f"four pages/{dtype}/{rid}")
    if dtype == "bfloat16":
        assert engine.graphs.replays > 100          # the single tokens ran as recorded steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_sizes_and_branches(tmp_path, dtype):
    """Widths that are no multiple of 8 or of 32, a latent too wide and heads too many for the matrix-core attention, a mLSTM
    key wider than 256, one stream, four streams, no logit scale, attention without a query factor, a layer that reads
    keys several layers back; prompts of more rows than the few-rows products take."""
    from kipp_amd.weights import write_random_model
    layers = [
        {"type": "attention", "mixer": {"heads": 18, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.3}, "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 40, "rot_dim": 24, "vdim": 12, "q_rank": 20, "kv_rank": 280, "scale": 0.05,
                                              "rot": {"base": 200.0, "dims": 24}, "mask": {"size": 100}}, "mlp": {"kind": "dense", "ff": 30}},
        {"type": "mlstm", "mixer": {"heads": 1, "dim": 260, "vdim": 20, "gate_cap": 3.0}, "mlp": {"kind": "dense", "ff": 52}},
        {"type": "attention", "mixer": {"heads": 18, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.2, "q_temp": {"coef": 2.0, "every": 100}, "kv_from": 0},
         "mlp": {"kind": "dense", "ff": 52}}]
    for streams, width in ((1, 100), (4, 72)):
        cfg = {"architecture": "Rerizen", "vocab": 77, "width": width, "streams": streams, "norm": {"eps": 1e-6}, "layers": layers}
        folder = write_random_model(str(tmp_path / f"odd{streams}"), cfg, seed=width, dtype=dtype)
        requests = {"long": H.random_tokens(1, 330, 77), "short": H.random_tokens(2, 9, 77)}
        for steps in (H.whole(requests), [([("long", 270)], []), ([("long", 59), ("short", 8)], []), ([("long", 1), ("short", 1)], ["long", "short"])]):
            got = H.replay(engine_of(folder, dtype), requests, steps)
            for rid, toks in requests.items():
                close(got[rid], plain_logits(folder, toks), TOL[dtype] * (4 if dtype == "bfloat16" else 1), f"{width}/{dtype}/{rid}")


def random_configuration(rng):
    """A model of the design with every size, the order of its layers and every constant drawn at random."""
    layers, sources = [], []
    for i in range(rng.randint(3, 6)):
        kind = rng.choice(["attention", "latent_attention", "mlstm"])
        mlp = None if rng.random() < 0.2 else {"kind": "dense", "ff": rng.choice([128, 200, 384])}
        if kind == "attention" and sources and rng.random() < 0.5:
            source = rng.choice(sources)
            mixer = dict(layers[source]["mixer"], scale=rng.uniform(0.05, 0.3), kv_from=source)
        elif kind == "attention":
            groups = rng.choice([1, 2, 3, 4])
            d = rng.choice([16, 32, 40, 64, 96])
            mixer = {"heads": groups * rng.choice([1, 2, 3]), "kv_heads": groups, "dim": d, "vdim": d if rng.random() < 0.5 else rng.choice([16, 24, 64]),
                     "scale": rng.uniform(0.05, 0.3)}
            if rng.random() < 0.7:
                mixer["q_temp"] = {"coef": rng.uniform(0.1, 1.0), "every": rng.choice([1, 7, 32, 64])}
            sources.append(i)
        elif kind == "latent_attention":
            dr = rng.choice([8, 16, 32])
            mixer = {"heads": rng.choice([2, 4, 6, 12, 20]), "dim": rng.choice([16, 32, 64]), "rot_dim": dr, "vdim": rng.choice([16, 32, 80]),
                     "q_rank": rng.choice([32, 64, 96]), "kv_rank": rng.choice([32, 48, 100, 128]), "scale": rng.uniform(0.05, 0.2),
                     "rot": {"base": rng.choice([10000.0, 500.0]), "dims": dr,
                             "scaling": {"factor": rng.choice([2.0, 8.0]), "original": rng.choice([64, 512]), "fast": 32.0, "slow": 1.0}},
                     "mask": {"size": rng.choice([1, 5, 16, 17, 64, 100, 300])}}
        else:
            mixer = {"heads": rng.choice([1, 2, 4]), "dim": rng.choice([16, 48, 64, 160]), "vdim": rng.choice([16, 48, 100]), "gate_cap": rng.choice([5.0, 15.0])}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Rerizen", "vocab": rng.choice([300, 512]), "width": rng.choice([96, 128, 192]), "streams": rng.choice([1, 2, 3, 4]),
            "logit_scale": rng.choice([0.25, 1.0, 3.0]), "norm": {"eps": rng.choice([1e-5, 1e-6])}, "layers": layers}


@pytest.mark.parametrize("seed", range(6))
def test_models_drawn_at_random(tmp_path, seed):
    """Sizes, order of layers and constants drawn at random; whole prompts, portions and mixed batches in float32."""
    import random

    from kipp_amd.weights import write_random_model
    cfg = random_configuration(random.Random(seed))
    folder = write_random_model(str(tmp_path / "drawn"), cfg, seed=seed, dtype="float32")
    requests = {f"r{i}": H.random_tokens(seed * 10 + i, n, cfg["vocab"]) for i, n in enumerate([1, 23, 97, 180])}
    for maker in (H.whole, H.changing_portions, lambda r: H.mixed(r, seed=seed)):
        got = H.replay(engine_of(folder, "float32", max_requests=4), requests, maker(requests))
        for rid, toks in requests.items():
            close(got[rid], plain_logits(folder, toks), 2e-8, f"drawn {seed}/{rid}: {json.dumps(cfg)}")


def test_recorded_steps_of_a_changing_batch(folders):
    """Three requests decode together from recorded steps while the window passes page borders and the memories go on in
    their slots; one ends early and the batch goes on at another size."""
    folder = folders[("rerizen-tiny-a", "bfloat16")]
    vocab = P.load_folder(folder)[0]["vocab"]
    requests = {"a": H.random_tokens(1, 90, vocab), "b": H.random_tokens(2, 120, vocab), "c": H.random_tokens(3, 75, vocab)}
    engine = engine_of(folder, "bfloat16")
    steps = [([("a", 30), ("b", 51), ("c", 2)], [])]
    fed = {"a": 30, "b": 51, "c": 2}
    while any(fed[r] < len(requests[r]) for r in fed):
        live = [r for r in fed if fed[r] < len(requests[r])]
        for r in live:
            fed[r] += 1
        steps.append(([(r, 1) for r in live], [r for r in live if fed[r] == len(requests[r])]))
    got = H.replay(engine, requests, steps)
    for rid, toks in requests.items():
        close(got[rid], plain_logits(folder, toks), TOL["bfloat16"], f"recorded/{rid}")
    assert engine.graphs.replays > 50


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(folders, dtype):
    """`generate` (scheduler, continuous batching, tokens chosen on the device) against the plain implementation:
    every generated token is the plain argmax of its position, or within rounding of it."""
    from kipp_amd import generate
    folder = folders[("rerizen-tiny-b", dtype)]
    cfg, w = P.load_folder(folder)
    prompts = [H.random_tokens(5, 3, cfg["vocab"]), H.random_tokens(6, 40, cfg["vocab"]), H.random_tokens(7, 21, cfg["vocab"])]
    outputs = generate(folder, prompts, max_new_tokens=30, dtype=dtype, page_size=16, prefill_chunk=16, max_step_tokens=24)
    margin = 1e-4 if dtype == "float32" else 0.05
    for prompt, out in zip(prompts, outputs):
        assert len(out) == 30
        logits = P.forward(cfg, w, prompt + out)
        for i, tok in enumerate(out):
            row = logits[len(prompt) - 1 + i]
            assert row[tok] >= row.max() - margin * (row.max() - row.min()), (dtype, i)


def test_trace_replay_and_command_line(folders, tmp_path):
    folder = folders[("rerizen-tiny-a", "bfloat16")]
    vocab = P.load_folder(folder)[0]["vocab"]
    toks = H.random_tokens(4, 60, vocab)
    lines = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[33:35], "want": []}, {"id": "y", "tokens": toks[:7], "want": [6]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[35:36], "want": [0]}], "end": ["x"]}]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "bfloat16", "--out", str(out),
                          "--max-tokens", "128"], input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = plain_logits(folder, toks)
    close(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, vocab), ref[[0, 32]], TOL["bfloat16"], "trace step 0")
    close(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, vocab), ref[[6]], TOL["bfloat16"], "trace step 1")
    close(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, vocab), ref[[35]], TOL["bfloat16"], "trace step 2")
    cli = subprocess.run([sys.executable, "-m", "kipp_amd.cli", "--model", folder, "--tokens", ",".join(map(str, toks[:9])), "--decode", "5"],
                         capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert cli.returncode == 0, cli.stderr[-2000:]
