"""The plain implementation of the Rerizen decoder pinned by hand, against second forms written another way, and the
design's configuration: keys, refusals, tensor names, what the cache manager is asked for.  No GPU."""
import copy
import math

import numpy as np
import pytest

from kipp_amd.config import ConfigError, parse_config, shape_config
from tests.plain import rerizen_plain as P


# ---- mechanisms by hand ------------------------------------------------------------------------------------

def test_masks_at_their_edges():
    w = P.windowed(9, 4)
    assert w[8, 5] and not w[8, 4] and w[8, 8] and not w[3, 4]          # itself and the three before it
    assert w[2].tolist() == [True, True, True] + [False] * 6             # the first tokens see all there is
    assert P.windowed(5, 1).tolist() == np.eye(5, dtype=bool).tolist()
    assert P.causal(4)[2].tolist() == [True, True, True, False]


def test_query_temperature_steps():
    f = P.query_temperature(13, 0.5, 4)
    assert f[0] == f[2] == 1.0                                           # floor((p + 1) / 4) = 0 up to p = 2
    assert f[3] == pytest.approx(1 + 0.5 * math.log(2)) and f[6] == f[3]
    assert f[7] == pytest.approx(1 + 0.5 * math.log(3)) and f[11] == pytest.approx(1 + 0.5 * math.log(4))


def test_rotary_frequencies_and_ramp():
    f, mag = P.rotary_frequencies(8, 100.0)
    assert mag == 1.0 and np.allclose(f, [1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75])
    sc = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    g, mag = P.rotary_frequencies(16, 10000.0, sc)
    plain = 10000.0 ** (-2.0 * np.arange(8) / 16)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    turn = lambda t: 16 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(turn(16.0)), 0), min(math.ceil(turn(2.0)), 15)
    assert (lo, hi) == (0, 2)
    assert g[0] == plain[0] and g[1] == pytest.approx(plain[1] * (0.5 / 4 + 0.5)) and np.allclose(g[2:], plain[2:] / 4)


def test_rotation_is_a_turn_of_interleaved_pairs():
    x = np.arange(12, dtype=float).reshape(2, 6) + 1
    f = np.array([0.3, 0.05, 1.1])
    y = P.rotate_pairs(x, [0, 5], f, 1.0)
    assert np.array_equal(y[0], x[0])                                    # position 0 turns nothing
    z = (x[1, 0::2] + 1j * x[1, 1::2]) * np.exp(1j * 5 * f)
    assert np.allclose(y[1, 0::2], z.real) and np.allclose(y[1, 1::2], z.imag)
    assert np.allclose(P.rotate_pairs(x, [0, 5], f, 1.25), 1.25 * y)


def test_streams_by_hand():
    X = np.array([[[1.0, 2.0]], [[10.0, 20.0]]])                         # two copies, one token, width 2
    assert np.array_equal(P.streams_read(X, [2.0, -1.0]), [[-8.0, -16.0]])
    M = np.array([[1.0, 3.0], [0.5, 0.0]])                               # [from, to]
    out = P.streams_write(X, M, [2.0, -1.0], np.array([[100.0, 200.0]]))
    assert np.array_equal(out[0], [[1 + 5 + 200, 2 + 10 + 400]]) and np.array_equal(out[1], [[3 - 100, 6 - 200]])


def _mlstm_case(seed=0, T=9, H=2, d=3, dv=4, width=5):
    rng = np.random.default_rng(seed)
    m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": 4.0}
    w = {"q": rng.normal(size=(H * d, width)), "k": rng.normal(size=(H * d, width)), "v": rng.normal(size=(H * dv, width)),
         "g": rng.normal(size=(H * dv, width)), "o": rng.normal(size=(width, H * dv)), "norm": 1 + rng.normal(size=H * dv) * 0.1,
         "i": rng.normal(size=(H, width)), "i.b": rng.normal(size=H), "f": rng.normal(size=(H, width)), "f.b": rng.normal(size=H) + 2}
    return m, w, rng.normal(size=(T, width))


def test_mlstm_against_the_unstabilised_sum():
    """Without the running maximum the memory is S_t = sum_j (prod_{j<l<=t} F_l) I_j k_j v_j^T; the stabilised recurrence
    gives the same output wherever max(|n.q|, e^-m) e^m = max(|n~.q|, 1) in true gates (the 1e-6 apart)."""
    m, w, h = _mlstm_case()
    y, _ = P.mlstm(h, w, m, 1e-5, "")
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, d) / math.sqrt(d)
    k, v = (h @ w["k"].T).reshape(T, H, d), (h @ w["v"].T).reshape(T, H, dv)
    li = 4.0 * np.tanh((h @ w["i"].T + w["i.b"]) / 4.0)
    lf = 4.0 * np.tanh((h @ w["f"].T + w["f.b"]) / 4.0)
    lf = -np.log1p(np.exp(-lf))
    out = np.zeros((T, H, dv))
    for head in range(H):
        for t in range(T):
            S, n = np.zeros((d, dv)), np.zeros(d)
            for j in range(t + 1):
                g = math.exp(li[j, head] + lf[j + 1:t + 1, head].sum())
                S += g * np.outer(k[j, head], v[j, head])
                n += g * k[j, head]
            # m_t as the recurrence defines it (it starts at 0)
            mx = 0.0
            for j in range(t + 1):
                mx = max(lf[j, head] + mx, li[j, head])
            out[t, head] = (S.T @ q[t, head]) * math.exp(-mx) / (max(abs(n @ q[t, head]) * math.exp(-mx), math.exp(-mx)) + 1e-6)
    o = P.rms(out, 1e-5).reshape(T, H * dv) * w["norm"] * P.sigmoid(h @ w["g"].T)
    assert np.allclose(y, o @ w["o"].T, rtol=1e-9, atol=1e-12)


def test_mlstm_state_carries_across_a_cut():
    m, w, h = _mlstm_case(seed=3, T=12)
    whole, _ = P.mlstm(h, w, m, 1e-5, "")
    first, state = P.mlstm(h[:5], w, m, 1e-5, "")
    second, _ = P.mlstm(h[5:], w, m, 1e-5, "", state)
    assert np.allclose(np.concatenate([first, second]), whole, rtol=1e-12, atol=1e-14)


def test_latent_attention_equals_its_absorbed_form():
    """Scores and values through the cached latent alone: q_h . W_uk_h c = (W_uk_h^T q_h) . c, and
    sum_j p_j W_uv_h c_j = W_uv_h sum_j p_j c_j."""
    rng = np.random.default_rng(1)
    T, width = 11, 10
    m = {"heads": 3, "dim": 4, "rot_dim": 4, "vdim": 5, "q_rank": 6, "kv_rank": 7, "scale": 0.3, "mask": {"size": 4},
         "rot": {"base": 50.0, "dims": 4, "scaling": {"factor": 3.0, "original": 8, "fast": 4.0, "slow": 1.0}}}
    w = {"dq": rng.normal(size=(6, width)), "dq.norm": 1 + rng.normal(size=6) * 0.1, "uq": rng.normal(size=(3 * 8, 6)),
         "dkv": rng.normal(size=(11, width)), "dkv.norm": 1 + rng.normal(size=7) * 0.1, "uk": rng.normal(size=(12, 7)),
         "uv": rng.normal(size=(15, 7)), "g": rng.normal(size=(3, width)), "o": rng.normal(size=(width, 15))}
    h = rng.normal(size=(T, width))
    y = P.latent_attention(h, w, m, 1e-5, "")
    cq = P.norm(h @ w["dq"].T, w["dq.norm"], 1e-5)
    q = (cq @ w["uq"].T).reshape(T, 3, 8)
    down = h @ w["dkv"].T
    c = P.norm(down[:, :7], w["dkv.norm"], 1e-5)
    f, mag = P.rotary_frequencies(4, 50.0, m["rot"]["scaling"])
    kr = P.rotate_pairs(down[:, 7:], np.arange(T), f, mag)
    out = np.zeros((T, 3, 5))
    for head in range(3):
        uk, uv = w["uk"][head * 4:(head + 1) * 4], w["uv"][head * 5:(head + 1) * 5]
        for i in range(T):
            ql = np.concatenate([uk.T @ q[i, head, :4], P.rotate_pairs(q[i:i + 1, head, 4:], [i], f, mag)[0]])
            js = [j for j in range(T) if 0 <= i - j < 4]
            s = np.array([ql @ np.concatenate([c[j], kr[j]]) for j in js]) * 0.3
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, head] = uv @ sum(pj * c[j] for pj, j in zip(p, js)) * P.sigmoid(h[i] @ w["g"][head])
    assert np.allclose(y, out.reshape(T, 15) @ w["o"].T, rtol=1e-9, atol=1e-12)


def test_attention_reads_another_layers_keys_and_a_changed_token_shows_causally():
    cfg = shape_config("rerizen-tiny-a")
    rng = np.random.default_rng(0)
    w = _random_weights(cfg, rng)
    toks = list(rng.integers(0, cfg["vocab"], 60))
    base = P.forward(cfg, w, toks)
    other = list(toks)
    other[30] = (other[30] + 1) % cfg["vocab"]
    changed = P.forward(cfg, w, other)
    assert np.array_equal(base[:30], changed[:30]) and not np.allclose(base[30:], changed[30:])
    # the layer that reads layer 1's keys has none of its own
    assert "l3.mix.k" not in w and "l3.mix.q" in w


def _random_weights(cfg, rng):
    from kipp_amd.engine.model import model_params
    spec = parse_config(cfg)[1].model_spec()
    return {name: (rng.normal(size=p.shape) * (0.3 if len(p.shape) == 2 else 0.1) + (1.0 if p.init[0] == "one_plus_normal" else 0.0)
                   + (np.eye(*p.shape) if p.init[0] == "eye_plus_normal" else 0.0)) for name, p in model_params(spec).items()}


def test_a_window_shows_exactly_at_its_edge():
    """One layer of latent attention with a window of 6: a changed token moves the logits of the five positions after it
    and of no later one."""
    cfg = {"architecture": "Rerizen", "vocab": 50, "width": 16, "streams": 2, "norm": {"eps": 1e-5}, "layers": [
        {"type": "latent_attention", "mlp": None, "mixer": {"heads": 2, "dim": 4, "rot_dim": 4, "vdim": 4, "q_rank": 8, "kv_rank": 6,
                                                           "scale": 0.5, "rot": {"base": 100.0, "dims": 4}, "mask": {"size": 6}}}]}
    rng = np.random.default_rng(5)
    w = _random_weights(cfg, rng)
    toks = list(rng.integers(0, 50, 30))
    other = list(toks)
    other[10] = (other[10] + 7) % 50
    a, b = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    moved = [i for i in range(30) if not np.array_equal(a[i], b[i])]
    assert moved == [10, 11, 12, 13, 14, 15]


# ---- configuration -------------------------------------------------------------------------------------------

def test_configuration_builds_the_model_as_data():
    from kipp_amd.engine.model import model_params
    from kipp_amd.parts import part_class
    cfg = shape_config("rerizen-tiny-a")
    family, typed = parse_config(cfg)
    spec = typed.model_spec()
    assert family.name == "Rerizen" and spec.streams == 3 and spec.head.scale == 0.5 and not spec.head.tied
    assert [layer.block for layer in spec.layers] == ["hyper_pre_norm", "hyper_pre_norm_mixer", "hyper_pre_norm", "hyper_pre_norm"]
    assert [run.cache_of for run in spec.order] == [None, None, None, 1]
    names = model_params(spec)
    assert names["l0.hc1.mix"].shape == (3, 3) and names["l2.mix.dkv"].shape == (48 + 16, 128) and names["l1.mix.q.b"].shape == (128,)
    assert "l3.mix.k" not in names and "l3.mix.v.b" not in names and "l1.norm2" not in names and "head" in names
    latent = spec.layers[2].part("mixer")
    need = part_class("mixer", "latent_attention").need_of(latent)
    assert (need.num_kv_heads, need.head_dim, need.value_dim, need.window) == (1, 64, 0, 40)
    assert parse_config(typed.to_dict())[1] == typed


def test_a_layer_that_reads_anothers_keys_may_leave_their_sizes_out():
    cfg = shape_config("rerizen-tiny-a")
    for key in ("kv_heads", "dim", "vdim"):
        del cfg["layers"][3]["mixer"][key]
    mixer = parse_config(cfg)[1].model_spec().layers[3].part("mixer")
    assert (mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, mixer.own_kv) == (2, 32, 32, False)


def test_configuration_without_streams_is_one_plain_residual():
    from kipp_amd.engine.model import model_params
    cfg = shape_config("rerizen-tiny-b")
    del cfg["streams"]
    spec = parse_config(cfg)[1].model_spec()
    assert spec.streams == 1 and not any(".hc" in name for name in model_params(spec))


@pytest.mark.parametrize("path, value, word", [
    (("layers", 0, "type"), "conv", "mixer of this design"),
    (("layers", 2, "mixer", "mask", "keep_first"), 2, "not implemented"),
    (("layers", 1, "mixer", "rot"), {"base": 10.0, "dims": 8}, "not implemented"),
    (("layers", 3, "mixer", "kv_from"), 2, "no keys and values"),
    (("layers", 3, "mixer", "kv_from"), 3, "earlier"),
    (("layers", 3, "mixer", "heads"), 8, "other head counts"),
    (("layers", 0, "mlp", "kind"), "routed", "feed-forward of this design"),
    (("layers", 2, "mixer", "rot", "dims"), 18, "exceeds"),
    (("streams",), 9, "streams"),
    (("layers", 0, "mixer", "gate_cap"), 0.0, "gate_cap"),
])
def test_refusals(path, value, word):
    cfg = shape_config("rerizen-tiny-a")
    at = cfg
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        parse_config(cfg)


def test_cache_manager_gets_a_group_a_need_and_a_slot_for_the_memory():
    from kipp_amd.cache import CacheManager
    from kipp_amd.cache.needs import StateNeed
    from kipp_amd.parts import part_class
    spec = parse_config(shape_config("rerizen-tiny-a"))[1].model_spec()
    needs, states = [], []
    for run in spec.order:
        mixer = spec.layers[run.layer].part("mixer")
        need_of = getattr(part_class("mixer", mixer.kind), "need_of", None)
        needs.append(need_of(mixer) if need_of is not None and run.cache_of is None else None)
        states.append(StateNeed((10,)) if mixer.kind == "mlstm" else None)
    manager = CacheManager(needs, states, 16, 8, 2, 4096, runtime=None)
    assert [g.runs for g in manager.groups] == [[1], [2]] and not manager.share        # the run that reads run 1's cache has none
    assert manager.groups[1].need.window == 40 and list(manager.state_needs) == [0]
    req = manager.open("a")
    manager.reserve([(req, 100)])
    manager.commit(req, [0] * 100)
    assert sum(p >= 0 for p in req.tables[1]) == 4 and sum(p >= 0 for p in req.tables[0]) == 7    # the window gave pages back
    manager.close("a")
    manager.check()
