"""Pins of the plain Tobinex implementation (hand-computed cases, invariants, a second scalar form), the
architecture's configuration, and the cache manager's bookkeeping of kept first pages.  No GPU."""
import math

import numpy as np
import pytest

from tests.plain import tobinex_plain as P


# ------------------------------------------------------------------------------- mechanisms, by hand

def test_mask_window_edge_and_kept_first():
    m = P.visible(12, size=4, keep_first=2)
    assert m[10, 10] and m[10, 7] and not m[10, 6]          # 10 - 7 = 3 < 4, 10 - 6 = 4 is outside
    assert m[10, 0] and m[10, 1] and not m[10, 2]           # the kept first two, and no third
    assert not m[3, 4]                                       # nothing ahead
    assert m[3, 0] and m[3, 3]                               # the first rows see everything behind them
    full = P.visible(6, size=None, keep_first=0)
    assert (full == np.tril(np.ones((6, 6), dtype=bool))).all()
    assert P.visible(9, size=1, keep_first=0).sum() == 9     # a window of one: only itself


def test_distance_bias_by_hand():
    b = P.distance_bias(4, [2.0], [0.5])
    assert b[0, 3, 3] == 0.0
    assert b[0, 3, 1] == pytest.approx(2.0 * math.log(1 + 0.5 * 2))
    assert b[0, 2, 0] == pytest.approx(2.0 * math.log(2.0))


def test_sink_joins_the_denominator_once():
    with np.errstate(divide="ignore"):
        scores = np.log(np.array([[[1.0, 0.0, 0.0], [1.0, 3.0, 0.0], [1.0, 3.0, 4.0]]]))    # exp(score) = 1, 3, 4
        p = P.sink_softmax(scores, P.visible(3, None, 0), [math.log(2.0)])
    assert p[0, 0] == pytest.approx([1 / 3, 0, 0])
    assert p[0, 2] == pytest.approx([1 / 10, 3 / 10, 4 / 10])
    assert p[0, 1].sum() == pytest.approx(4 / 6)            # the sink takes its share and has no value
    q = P.sink_softmax(scores, P.visible(3, None, 0), [-np.inf])
    assert q[0, 2].sum() == pytest.approx(1.0)


def test_heads_are_mixed_after_the_softmax():
    p = np.arange(2 * 3 * 3, dtype=float).reshape(2, 3, 3)
    out = P.mix_heads(p, [[1.0, 0.5], [-2.0, 0.0]])
    assert (out[0] == p[0] + 0.5 * p[1]).all() and (out[1] == -2.0 * p[0]).all()
    assert (P.mix_heads(p, np.eye(2)) == p).all()


def test_norms():
    x = np.array([[3.0, 4.0]])
    assert P.rms(x, 0.0)[0] == pytest.approx([3 / math.sqrt(12.5), 4 / math.sqrt(12.5)])
    assert P.one_plus_norm(x, [0.0, 1.0], 0.0)[0] == pytest.approx([3 / math.sqrt(12.5), 8 / math.sqrt(12.5)])
    assert P.plain_weight_norm(x, [0.0, 1.0], 0.0)[0] == pytest.approx([0.0, 4 / math.sqrt(12.5)])
    assert P.rms(np.zeros((1, 4)), 1e-6)[0] == pytest.approx([0, 0, 0, 0])     # eps inside the root


def test_embedding_scale_and_head_without_it():
    table = np.array([[1.0, 2.0], [3.0, -1.0]])
    assert (P.embed(table, [1, 0], 2.0) == [[6.0, -2.0], [2.0, 4.0]]).all()


# ------------------------------------------------------------------------------- a second form, written on its own

def _attention_loops(x, w, m, eps):
    """One query at a time, scalar loops, a running list of keys: nothing shared with P.attention but the inputs."""
    T = x.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size = (m.get("mask") or {}).get("size")
    keep = (m.get("mask") or {}).get("keep_first", 0)
    keys, values, out = [], [], np.zeros((T, H * dv))
    for i in range(T):
        q = w["q"] @ x[i]
        q = q / math.sqrt(float(np.mean(q * q)) + eps) * w["q.norm"]
        k = w["k"] @ x[i]
        keys.append(k / math.sqrt(float(np.mean(k * k)) + eps) * w["k.norm"])
        values.append(w["v"] @ x[i])
        seen = [j for j in range(i + 1) if size is None or i - j < size or j < keep]
        weights = np.zeros((H, len(seen)))
        for h in range(H):
            c = h // (H // G)
            e = [math.exp(m["scale"] * float(q[h * d:(h + 1) * d] @ keys[j][c * d:(c + 1) * d])
                          - w["r1"][h] * math.log(1 + w["r2"][h] * (i - j))) for j in seen]
            weights[h] = np.array(e) / (math.exp(w["sink"][h]) + sum(e))
        mixed = w["talk"] @ weights
        gate = 1.0 / (1.0 + np.exp(-(w["g"] @ x[i])))
        for h in range(H):
            c = h // (H // G)
            o = sum(mixed[h, n] * values[j][c * dv:(c + 1) * dv] for n, j in enumerate(seen))
            out[i, h * dv:(h + 1) * dv] = o * gate[h * dv:(h + 1) * dv]
    return out @ w["o"].T


@pytest.mark.parametrize("mask", [{"size": 5, "keep_first": 2}, {"size": 3, "keep_first": 0}, None])
def test_attention_agrees_with_its_scalar_form(mask):
    rng = np.random.default_rng(5)
    H, G, d, dv, width, T = 4, 2, 6, 3, 10, 14
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": 0.7, "mask": mask}
    w = {"q": rng.normal(size=(H * d, width)), "k": rng.normal(size=(G * d, width)), "v": rng.normal(size=(G * dv, width)),
         "g": rng.normal(size=(H * dv, width)), "o": rng.normal(size=(width, H * dv)),
         "q.norm": rng.normal(size=H * d) + 1, "k.norm": rng.normal(size=G * d) + 1, "r1": np.abs(rng.normal(size=H)),
         "r2": np.abs(rng.normal(size=H)), "sink": rng.normal(size=H), "talk": rng.normal(size=(H, H))}
    x = rng.normal(size=(T, width))
    assert np.allclose(P.attention(x, w, m, 1e-5), _attention_loops(x, w, m, 1e-5), rtol=1e-10, atol=1e-12)


def _random_model(cfg, seed):
    rng = np.random.default_rng(seed)
    width = cfg["width"]
    w = {"embed": rng.normal(size=(cfg["vocab"], width)) * 0.1, "final.norm": rng.normal(size=width) * 0.2}
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = f"l{i}."
        w.update({p + "norm1": rng.normal(size=width) * 0.2, p + "mix.q": rng.normal(size=(H * d, width)) * 0.2,
                  p + "mix.k": rng.normal(size=(G * d, width)) * 0.2, p + "mix.v": rng.normal(size=(G * dv, width)) * 0.2,
                  p + "mix.g": rng.normal(size=(H * dv, width)) * 0.2, p + "mix.o": rng.normal(size=(width, H * dv)) * 0.2,
                  p + "mix.q.norm": rng.normal(size=H * d) * 0.3 + 1, p + "mix.k.norm": rng.normal(size=G * d) * 0.3 + 1,
                  p + "mix.r1": np.abs(rng.normal(size=H)), p + "mix.r2": np.abs(rng.normal(size=H)) * 0.3,
                  p + "mix.sink": rng.normal(size=H), p + "mix.talk": rng.normal(size=(H, H)) * 0.5})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            w.update({p + "norm2": rng.normal(size=width) * 0.2, p + "mlp.gate": rng.normal(size=(ff, width)) * 0.2,
                      p + "mlp.up": rng.normal(size=(ff, width)) * 0.2, p + "mlp.down": rng.normal(size=(width, ff)) * 0.2})
    return w


def test_a_position_does_not_depend_on_what_follows():
    from kipp_amd.config import shape_config
    cfg = shape_config("tobinex-tiny-a")
    w = _random_model(cfg, 3)
    tokens = list(np.random.default_rng(1).integers(0, cfg["vocab"], size=50))
    whole = P.forward_whole(cfg, w, tokens)
    assert np.allclose(P.forward_whole(cfg, w, tokens[:31]), whole[:31], rtol=1e-9, atol=1e-11)
    layers = []
    P.forward_whole(cfg, w, tokens[:5], layers)
    assert len(layers) == len(cfg["layers"]) and layers[0].shape == (5, cfg["width"])


def test_the_window_changes_the_result_exactly_where_it_should():
    """A key one step outside the window must not matter; one step inside must."""
    from kipp_amd.config import shape_config
    cfg = shape_config("tobinex-tiny-a")
    cfg["layers"] = cfg["layers"][:1]                      # window 24, the first 3 kept
    w = _random_model(cfg, 4)
    base = [int(t) for t in np.random.default_rng(2).integers(0, cfg["vocab"], size=40)]
    ref = P.forward_whole(cfg, w, base)[39]
    for at, matters in ((15, False), (16, True), (3, False), (2, True)):     # 39 - 15 = 24 is outside, 39 - 16 = 23 inside
        other = list(base)
        other[at] = (base[at] + 1) % cfg["vocab"]
        got = P.forward_whole(cfg, w, other)[39]
        assert (np.abs(got - ref).max() > 1e-9) == matters, at


# ------------------------------------------------------------------------------- configuration and registry

def test_configuration_is_read_from_its_keys():
    from kipp_amd.config import parse_config, shape_config
    from kipp_amd.engine.model import model_params
    d = shape_config("tobinex-tiny-b")
    family, cfg = parse_config(d)
    assert family.name == "Tobinex" and cfg.to_dict() == d
    spec = cfg.model_spec()
    assert [layer.block for layer in spec.layers] == ["post_norm"] * 3 and spec.layers[0].residual_scale == 1.7
    mixer = spec.layers[1].part("mixer")
    assert (mixer.num_heads, mixer.num_kv_heads, mixer.head_dim, mixer.v_head_dim, mixer.window, mixer.keep_first) == (12, 4, 32, 64, 33, 1)
    names = model_params(spec)
    assert names["l1.mix.talk"].shape == (12, 12) and names["l0.mix.q.norm"].shape == (120,) and names["embed"].shape == (131, 80)
    assert names["l2.mix.o"].shape == (80, 32) and names["l0.mlp.down"].shape == (80, 56) and "final.norm" in names
    a = parse_config(shape_config("tobinex-tiny-a"))[1].model_spec()
    assert a.layers[1].block == "post_norm_mixer" and "l1.norm2" not in model_params(a) and "l1.mlp.up" not in model_params(a)
    assert a.layers[2].part("mixer").window is None and a.head.tied and a.embedding.scale == 9.8


@pytest.mark.parametrize("change, match", [
    (lambda d: d["layers"][0].update(type="recurrent"), "type"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda d: d["layers"][1]["mixer"].update(kv_heads=5), "multiple"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d.pop("postln_alpha"), "postln_alpha"),
    (lambda d: d["norm"].update(eps=-1.0), "eps"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda d: d.update(layers=[]), "layers"),
])
def test_what_is_not_implemented_is_refused(change, match):
    from kipp_amd.config import ConfigError, parse_config, shape_config
    d = shape_config("tobinex-tiny-b")
    change(d)
    with pytest.raises(ConfigError, match=match):
        parse_config(d)


def test_random_model_folder_round_trip(tmp_path):
    from kipp_amd.config import shape_config
    from kipp_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "m"), shape_config("tobinex-tiny-a"), seed=5, dtype="bfloat16")
    cfg, w = P.load_folder(folder)
    assert w["l0.mix.r2"].min() >= 0 and w["l2.mix.talk"].shape == (4, 4)
    logits = P.forward_whole(cfg, w, [1, 2, 3, 4])
    assert logits.shape == (4, 193) and np.isfinite(logits).all()


# ------------------------------------------------------------------------------- pages of the kept first keys

def test_a_window_gives_pages_back_but_never_the_kept_first_ones():
    from kipp_amd.cache import CacheManager
    from kipp_amd.cache.needs import KVNeed
    need = KVNeed(num_kv_heads=2, head_dim=8, window=10, page_size=None, v_head_dim=4, keep_first=5)
    plain_need = KVNeed(num_kv_heads=2, head_dim=8, window=10)
    cm = CacheManager([need, plain_need], [None, None], page_size=4, num_pages=12, max_requests=2, max_position=200)
    kept, gone = cm.groups
    assert kept.kept_blocks() == 2 and gone.kept_blocks() == 0
    assert kept.bytes_per_token(2) == 2 * (8 + 4) * 2
    req = cm.open("a")
    for _ in range(40):
        cm.reserve([(req, 1)])
        cm.commit(req, [7])
        cm.check()
    table = req.tables[kept.index]
    assert table[0] >= 0 and table[1] >= 0                   # positions 0 .. 4 lie in blocks 0 and 1
    first_needed = (40 - 10 + 1) // 4
    assert all(p < 0 for p in table[2:first_needed]) and all(p >= 0 for p in table[first_needed:])
    assert all(p < 0 for p in req.tables[gone.index][:first_needed])
    # what a scheduler keeps free for a request counts the kept blocks too
    assert cm.pages_bound(None, 1000, 1)[kept.index] == cm.pages_bound(None, 1000, 1)[gone.index] + 2
    cm.close("a")
    assert cm.free_pages() == [12, 12]
