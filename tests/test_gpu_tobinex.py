"""The Tobinex design on the GPU against its plain implementation: every kernel of the mixer alone (each mechanism
switched on and off, crafted keys at every edge), then the engine under every cutting in both precisions, tight
pools, long decoding, recorded steps, generation through the scheduler, the trace replay and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers as H
from tests.plain import tobinex_plain as P

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHAPES = ("tobinex-tiny-a", "tobinex-tiny-b")
LENGTHS = [1, 19, 45, 80, 131]
TOL = {"float32": 1e-10, "bfloat16": 2e-4}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    root = tmp_path_factory.mktemp("tobinex")
    return {(shape, dtype): write_random_model(str(root / f"{shape}-{dtype}"), shape_config(shape), seed=40 + i, dtype=dtype)
            for i, shape in enumerate(SHAPES) for dtype in ("float32", "bfloat16")}


_plain_cache = {}


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        cfg, w = P.load_folder(folder)
        _plain_cache[key] = P.forward_whole(cfg, w, list(tokens))
    return _plain_cache[key]


def close(got, ref, tol, what):
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    worst = max(float(np.sum((g - r) ** 2) / np.sum(r ** 2)) for g, r in zip(got.astype(np.float64), ref))
    assert worst <= tol, f"{what}: NMSE {worst:.3e} exceeds {tol:.1e}"


def engine_of(folder, dtype, page=16, **kw):
    from kipp_amd.engine import Engine
    kw.setdefault("max_tokens", 1024)
    return Engine.from_folder(folder, dtype=dtype, page_size=page, share_prefixes=False, **kw)


# =============================================================================== the mixer's kernels alone

def bf16(x):
    import torch
    return torch.tensor(np.asarray(x, dtype=np.float32)).bfloat16().float().numpy().astype(np.float64)


class MixerCase:
    """One sequence of T tokens whose projections are given; the kernels norm q and k, fill the pages (handed out in a
    scrambled order) and attend; the same from the plain functions.  `queries`: None = all T rows as one prompt
    portion; a list of positions = each as a single decoded token of an entry of its own that shares the pages."""

    def __init__(self, H_, G, d, dv, window, keep, T, seed=0, page=16, bias=True, sink=True, mix=True, gate=True):
        rng = np.random.default_rng(seed)
        self.H, self.G, self.d, self.dv, self.window, self.keep, self.T, self.page = H_, G, d, dv, window, keep, T, page
        self.width = H_ * d + G * d + G * dv + H_ * dv
        self.proj = rng.normal(size=(T, self.width)).astype(np.float32)
        self.qw = (rng.normal(size=H_ * d) * 0.3 + 1).astype(np.float32)
        self.kw = (rng.normal(size=G * d) * 0.3 + 1).astype(np.float32)
        self.r1 = np.abs(rng.normal(size=H_)).astype(np.float32) if bias else None
        self.r2 = (np.abs(rng.normal(size=H_)) * 0.3).astype(np.float32) if bias else None
        self.sink = rng.normal(size=H_).astype(np.float32) if sink else None
        self.mix = (rng.normal(size=(H_, H_)) * 0.5 + np.eye(H_)).astype(np.float32) if mix else None
        self.gate = gate
        self.scale, self.eps = 0.37, 1e-5

    def stand_out(self, key, strength=30.0):
        """Key `key` of every key/value head points where every query points, far longer than the others: wherever
        it is seen it takes the softmax, and its value (a constant far from the others) the output."""
        H_, G, d, dv = self.H, self.G, self.d, self.dv
        u = np.ones(d, dtype=np.float32)
        for h in range(H_):
            self.proj[:, h * d:(h + 1) * d] += 6.0 * u
        for c in range(G):
            self.proj[key, H_ * d + c * d:H_ * d + (c + 1) * d] = strength * u
            self.proj[key, H_ * d + G * d + c * dv:H_ * d + G * d + (c + 1) * dv] = 200.0
        return self

    def plain(self, rounded):
        H_, G, d, dv, T = self.H, self.G, self.d, self.dv, self.T
        x = self.proj.astype(np.float64)
        q = P.plain_weight_norm(x[:, :H_ * d], self.qw, self.eps)
        k = P.plain_weight_norm(x[:, H_ * d:H_ * d + G * d], self.kw, self.eps)
        v = x[:, H_ * d + G * d:H_ * d + G * d + G * dv]
        if rounded:
            q, k, v = bf16(q), bf16(k), bf16(v)
        kv_of = np.arange(H_) // (H_ // G)
        s = np.einsum("ihd,jhd->hij", q.reshape(T, H_, d), k.reshape(T, G, d)[:, kv_of]) * self.scale
        if self.r1 is not None:
            s = s - P.distance_bias(T, self.r1, self.r2)
        p = P.sink_softmax(s, P.visible(T, self.window, self.keep), self.sink if self.sink is not None else np.full(H_, -np.inf))
        if self.mix is not None:
            p = P.mix_heads(p, self.mix)
        o = np.einsum("hij,jhe->ihe", p, v.reshape(T, G, dv)[:, kv_of]).reshape(T, H_ * dv)
        if self.gate:
            o = o * P.sigmoid(x[:, H_ * d + G * d + G * dv:])
        return o

    def run(self, dtype, fast, queries=None, slabs=1):
        import torch
        from kipp_amd.csrc import ops
        dev = torch.device("cuda:0")
        H_, G, d, dv, T, page = self.H, self.G, self.d, self.dv, self.T, self.page
        t = lambda a, ty=None: None if a is None else torch.tensor(a, device=dev, dtype=ty)
        act = torch.float32 if dtype == "float32" else torch.bfloat16
        blocks = -(-T // page)
        pages = np.random.default_rng(9).permutation(blocks + 3)[:blocks].astype(np.int32)      # scrambled, with holes
        k_cache = torch.full((blocks + 3, G, page, d), 7.0, dtype=act, device=dev)             # stale values everywhere
        v_cache = torch.full((blocks + 3, G, page, dv), -3.0, dtype=act, device=dev)
        proj = t(self.proj)
        if slabs > 1:           # the same sum, as a split product hands it over
            parts = torch.randn((slabs - 1,) + proj.shape, device=dev)
            proj = torch.cat([parts, (proj - parts.sum(0)).unsqueeze(0)], 0).contiguous()
        i32 = torch.int32
        positions, seq = t(np.arange(T), i32), torch.zeros(T, dtype=i32, device=dev)
        table = t(pages[None, :], i32)
        q = ops.mixed_prepare(proj, torch.empty((T, H_ * d), dtype=act, device=dev), k_cache, v_cache, positions, seq, table,
                              H_, G, d, dv, t(self.qw), t(self.kw), self.eps)
        if queries is None:
            rows, q_rows, gate_rows = np.arange(T), q, proj
            q_start, q_len, ctx_len, tables = [0], [T], [T], table
        else:
            rows = np.asarray(queries)
            idx = t(rows, torch.int64)
            q_rows = q[idx].contiguous()
            gate_rows = proj[..., idx, :].contiguous()
            q_start, q_len, ctx_len = list(range(len(rows))), [1] * len(rows), [int(r) + 1 for r in rows]
            tables = table.repeat(len(rows), 1).contiguous()
            positions, seq = t(rows, i32), t(np.arange(len(rows)), i32)
        n = len(rows)
        out = torch.empty((n, H_ * dv), dtype=act, device=dev)
        gate_at = H_ * d + G * d + G * dv
        common = (H_, G, d, dv, self.scale, self.window or 0, self.keep, t(self.r1), t(self.r2), t(self.sink), t(self.mix))
        if not fast:
            ops.mixed_attention_plain(q_rows, k_cache, v_cache, out, positions, seq, tables, *common,
                                      gate=gate_rows if self.gate else None, gate_at=gate_at)
        else:
            assert ops.mixed_attention_fast_ok(H_, d, dv, page)
            entry, row0, split, nsplits, row_splits = [], [], [], [], []
            for e, (m, ctx) in enumerate(zip(q_len, ctx_len)):
                for r0 in range(0, m, 16):
                    runs = 1 + (e + r0 // 16) % 3           # one, two or three runs of keys, in turn
                    entry += [e] * runs
                    row0 += [r0] * runs
                    split += list(range(runs))
                    nsplits += [runs] * runs
                    row_splits += [runs] * min(16, m - r0)
            space = ops.mixed_attention_workspace(len(entry), n, H_, dv, 3, dev)
            ops.mixed_attention_mfma(q_rows, k_cache, v_cache, out, tuple(t(a, i32) for a in (entry, row0, split, nsplits)),
                                     len(entry), t(row_splits, i32), 3, t(q_start, i32), t(q_len, i32), t(ctx_len, i32), tables,
                                     *common, space, gate=gate_rows if self.gate else None, gate_at=gate_at)
        torch.cuda.synchronize()
        return out.float().cpu().numpy(), rows


PATHS = [("float32", False), ("bfloat16", False), ("bfloat16", True)]
KERNEL_TOL = {"float32": 1e-10, "bfloat16": 1e-4}


@pytest.mark.parametrize("dtype, fast", PATHS)
@pytest.mark.parametrize("off", [None, "bias", "sink", "mix", "gate"])
def test_each_mechanism_alone_and_together(dtype, fast, off):
    """All four extras on, then each one off in turn: a kernel that ignored one, or applied it twice, shows."""
    flags = {name: name != off for name in ("bias", "sink", "mix", "gate")}
    case = MixerCase(6, 3, 32, 16, window=21, keep=4, T=70, seed=3, **flags)
    got, rows = case.run(dtype, fast)
    close(got, case.plain(dtype == "bfloat16")[rows], KERNEL_TOL[dtype], f"{dtype}/{fast}/without {off}")


@pytest.mark.parametrize("dtype, fast", PATHS)
@pytest.mark.parametrize("geometry", [(4, 4, 32, 32, None, 0), (8, 2, 64, 48, 40, 0), (12, 4, 32, 64, 33, 1), (2, 1, 96, 16, 16, 20),
                                      (32, 8, 32, 16, 50, 2), (5, 5, 24, 20, 17, 9), (3, 1, 40, 8, 1, 0)])
def test_geometries_prompt_and_single_tokens(dtype, fast, geometry):
    """Head counts, groupings and sizes (keys and values of different widths), no window, a window of one, more kept
    keys than the window is long; rows as one prompt and as single tokens anywhere in the sequence, the projections
    in slabs."""
    from kipp_amd.csrc import ops
    H_, G, d, dv, window, keep = geometry
    if fast and not ops.mixed_attention_fast_ok(H_, d, dv, 16):
        pytest.skip("the matrix-core form does not take these sizes; the plain form is what runs")
    case = MixerCase(H_, G, d, dv, window, keep, T=150, seed=H_)
    ref = case.plain(dtype == "bfloat16")
    got, rows = case.run(dtype, fast, slabs=3)
    close(got, ref[rows], KERNEL_TOL[dtype], f"prompt {geometry}")
    got, rows = case.run(dtype, fast, queries=[0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 100, 127, 128, 149])
    close(got, ref[rows], KERNEL_TOL[dtype], f"single tokens {geometry}")


@pytest.mark.parametrize("dtype, fast", PATHS)
@pytest.mark.parametrize("page", [16, 32])
def test_a_key_that_stands_out_at_every_edge(dtype, fast, page):
    """One key far longer than the rest, placed in turn just inside and just outside the window of the query that is
    asked, among the kept first keys and right behind them, far back, and on both sides of page and tile borders: seen
    where it must not be, or missed, the output changes altogether."""
    window, keep, T = 37, 5, 200
    for query in (199, 160, 96, 41):
        edges = {query - window + 1, query - window, keep - 1, keep, 0, query, query - 1,
                 (query - window + 1) // page * page, (query - window + 1) // page * page - 1, 31, 32, 2}
        for key in sorted(k for k in edges if 0 <= k <= query):
            case = MixerCase(4, 2, 32, 16, window, keep, T, seed=key, page=page).stand_out(key)
            ref = case.plain(dtype == "bfloat16")
            seen = query - key < window or key < keep
            assert (np.abs(ref[query]).max() > 20.0) == seen      # the crafted value shows exactly where the key is seen
            got, rows = case.run(dtype, fast, queries=[query])
            close(got, ref[rows], KERNEL_TOL[dtype] * 10, f"single token {query}, key {key}")
            got, rows = case.run(dtype, fast)
            close(got[query:query + 1], ref[query:query + 1], KERNEL_TOL[dtype] * 10, f"prompt row {query}, key {key}")


def test_post_norm_and_scaled_embedding_kernels():
    import torch
    from kipp_amd.csrc import ops
    rng = np.random.default_rng(0)
    for width in (80, 96, 1000):
        x = rng.normal(size=(7, width)).astype(np.float32)
        delta = rng.normal(size=(3, 7, width)).astype(np.float32)
        w = rng.normal(size=width).astype(np.float32)
        ref = P.rms(2.5 * x.astype(np.float64) + delta.astype(np.float64).sum(0), 1e-5) * w
        xd = torch.tensor(x, device="cuda")
        rows = torch.empty((7, width), dtype=torch.bfloat16, device="cuda")
        ops.scaled_add_rmsnorm(xd, torch.tensor(delta, device="cuda"), 2.5, torch.tensor(w, device="cuda"), 1e-5, rows)
        assert np.allclose(xd.cpu().numpy(), ref, rtol=2e-6, atol=2e-6)
        assert (rows.float().cpu().numpy() == xd.bfloat16().float().cpu().numpy()).all()      # the same rows, rounded once
    table = torch.tensor(rng.normal(size=(11, 24)).astype(np.float32), device="cuda").bfloat16()
    out = ops.embed_scaled(table, torch.tensor([3, 0, 10], dtype=torch.int32, device="cuda"), torch.empty((3, 24), device="cuda"), 6.25)
    assert (out.cpu().numpy() == table.float().cpu().numpy()[[3, 0, 10]] * np.float32(6.25)).all()


# =============================================================================== the engine

def requests_of(vocab, seed=0, lengths=LENGTHS):
    return {f"r{i}": H.random_tokens(seed * 100 + i, n, vocab) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype, page", [("float32", 16), ("bfloat16", 16), ("bfloat16", 32), ("bfloat16", 8)])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuttings_match_plain(folders, shape, dtype, page, cut):
    """Whole prompts, the last tokens one by one, portions of changing size down to two tokens, and mixed batches in a
    pool that only holds the live requests (pages and slots are used again).  Pages of 8 run the plain kernels under
    bfloat16, 16 and 32 the matrix-core ones."""
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
    assert (engine.rt.generic_attention_launches > 0) == (dtype == "bfloat16" and (page == 8 or shape == "tobinex-tiny-b"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width, ff, heads", [(100, 52, (3, 1, 20, 12)), (72, 200, (2, 2, 36, 28)), (160, 88, (16, 4, 32, 16))])
def test_sizes_that_leave_the_fast_kernels(tmp_path, dtype, width, ff, heads):
    """Widths that are no multiple of 8 or of 32 (their products go to other kernels or to the library's), head sizes
    only the plain attention takes, prompts longer than the few-rows and staged-rows products take, a vocabulary that is
    no multiple of anything."""
    from kipp_amd.weights import write_random_model
    H_, G, d, dv = heads
    cfg = {"architecture": "Tobinex", "vocab": 77, "width": width, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5}, "postln_alpha": 0.8,
           "layers": [{"type": "attention", "mlp": {"kind": "dense", "ff": ff},
                       "mixer": {"heads": H_, "kv_heads": G, "dim": d, "vdim": dv, "scale": 0.3, "mask": {"size": 50 + 7 * i, "keep_first": 2 * i}}}
                      for i in range(2)]}
    folder = write_random_model(str(tmp_path / "odd"), cfg, seed=width, dtype=dtype)
    requests = {"long": H.random_tokens(1, 330, 77), "short": H.random_tokens(2, 9, 77)}
    for steps in (H.whole(requests), [([("long", 270)], []), ([("long", 59), ("short", 8)], []), ([("long", 1), ("short", 1)], ["long", "short"])]):
        got = H.replay(engine_of(folder, dtype), requests, steps)
        for rid, toks in requests.items():
            close(got[rid], plain_logits(folder, toks), TOL[dtype], f"{width}/{dtype}/{rid}")


@pytest.mark.parametrize("shape", SHAPES)
def test_float32_cuttings_are_bitwise_equal(folders, shape):
    """In float32 every sum runs in an order that the token's own position fixes: how the prompt was cut, what else was
    in the batch and which pages were used change no bit."""
    folder = folders[(shape, "float32")]
    requests = requests_of(P.load_folder(folder)[0]["vocab"], seed=3)
    base = H.replay(engine_of(folder, "float32"), requests, H.whole(requests))
    for maker in (H.tail_one_by_one, H.changing_portions, lambda r: H.mixed(r, seed=11)):
        steps = maker(requests)
        order = list(np.random.default_rng(1).permutation(64))
        got = H.replay(engine_of(folder, "float32", page_order=order), requests, steps)
        for rid in requests:
            assert np.array_equal(got[rid], base[rid]), f"{shape}/{rid}: bits differ between cuttings"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_pool_of_four_pages(tmp_path, dtype):
    """A window of 20 with 3 kept keys in pages of 16: one kept page, two that the window covers and the one being
    filled.  200 tokens pass through those four pages; the kept page stays, the others come round again and again."""
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    cfg = shape_config("tobinex-tiny-a")
    cfg["layers"] = [cfg["layers"][0]]
    cfg["layers"][0]["mixer"]["mask"] = {"size": 20, "keep_first": 3}
    folder = write_random_model(str(tmp_path / "one"), cfg, seed=8, dtype=dtype)
    tokens = H.random_tokens(77, 200, cfg["vocab"])
    engine = engine_of(folder, dtype, 16, max_tokens=None, num_pages=4, max_requests=2)
    steps = [([("r", 10)], [])] + [([("r", 1)], []) for _ in range(60)] + [([("r", 7)], []), ([("r", 2)], [])] \
        + [([("r", 1)], []) for _ in range(121)]
    steps[-1] = (steps[-1][0], ["r"])
    got = H.replay(engine, {"r": tokens}, steps)
    close(got["r"], plain_logits(folder, tokens), TOL[dtype], f"four pages/{dtype}")
    if dtype == "bfloat16":
        assert engine.graphs.replays > 100          # the single tokens ran as recorded steps


def test_recorded_steps_of_a_changing_batch(folders):
    """Three requests decode together from recorded steps while their windows pass page borders; one ends early and
    the batch goes on at another size."""
    folder = folders[("tobinex-tiny-a", "bfloat16")]
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
    folder = folders[("tobinex-tiny-b", dtype)]
    cfg, w = P.load_folder(folder)
    prompts = [H.random_tokens(5, 3, cfg["vocab"]), H.random_tokens(6, 40, cfg["vocab"]), H.random_tokens(7, 21, cfg["vocab"])]
    outputs = generate(folder, prompts, max_new_tokens=30, dtype=dtype, page_size=16, prefill_chunk=16, max_step_tokens=24)
    margin = 1e-4 if dtype == "float32" else 0.05
    for prompt, out in zip(prompts, outputs):
        assert len(out) == 30
        logits = P.forward_whole(cfg, w, prompt + out)
        for i, tok in enumerate(out):
            row = logits[len(prompt) - 1 + i]
            assert row[tok] >= row.max() - margin * (row.max() - row.min()), (dtype, i)


def test_trace_replay_and_command_line(folders, tmp_path):
    folder = folders[("tobinex-tiny-a", "bfloat16")]
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
