"""The Tabatar design without a GPU: its configuration, its plan, the tensors and state it declares, and the plain
implementation's own mechanisms against independent formulas."""
import math

import numpy as np
import pytest

import plain_tabatar as pt
import tabatar_models as tm
from inferflux_amd.cache.storage import plan_groups
from inferflux_amd.config import ConfigError, config_from_dict, load_config, plan_for
from inferflux_amd.config.tabatar import TabatarConfig
from inferflux_amd.engine.model import Model


def test_config_reads_every_layer_and_roundtrips(tmp_path):
    for name in tm.CONFIGS:
        d = tm.config(name)
        cfg = config_from_dict(d)
        assert isinstance(cfg, TabatarConfig) and (cfg.vocab, cfg.width, cfg.norm_eps) == (d["vocab"], d["width"], d["norm"]["eps"])
        assert (cfg.embedding_scale, cfg.streams, cfg.logit_scale, cfg.logit_softcap) == \
               (d["embedding"]["scale"], d.get("streams"), d["logit_scale"], d.get("logit_softcap"))
        assert (cfg.loop is None) == ("loop" not in d)
        for L, want in zip(cfg.layers, d["layers"]):
            m = want["mixer"]
            assert L.type == want["type"] and (L.mlp is None) == (want["mlp"] is None)
            if L.type == "attention":
                assert (L.mixer.heads, L.mixer.kv_heads, L.mixer.dim, L.mixer.vdim, L.mixer.scale) == \
                       (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"])
                assert L.mixer.window == (m.get("mask") or {}).get("size")
                assert (L.mixer.rot_base, L.mixer.rot_dims) == (m["rot"]["base"], m["rot"]["dims"])
                assert (L.mixer.rot_scaling is None) == ("scaling" not in m["rot"])
            else:
                assert (L.mixer.heads, L.mixer.dim, L.mixer.vdim, L.mixer.tau, L.mixer.rank) == (m["heads"], m["dim"], m["vdim"], m["tau"], m["rank"])
            if want["mlp"] and want["mlp"]["kind"] == "moe":
                w = want["mlp"]
                assert (L.mlp.ff, L.mlp.experts, L.mlp.top, L.mlp.shared_ff) == \
                       (w["expert"]["ff"], w["router"]["experts"], w["router"]["top"], (w.get("shared") or {}).get("ff", 0))
        cfg.save(str(tmp_path / name))
        assert load_config(str(tmp_path / name)) == cfg


def test_keys_that_may_be_absent_have_their_meaning():
    d = tm.model(50, 32, 1e-5, [tm.layer(tm.attention(2, 2, 8, 8, 0.5, 100.0, 8), tm.dense(16))])
    for k in ("kv_heads", "vdim"):
        del d["layers"][0]["mixer"][k]
    del d["layers"][0]["mixer"]["rot"]["dims"]
    del d["embedding"], d["logit_scale"]
    cfg = config_from_dict(d)
    m = cfg.layers[0].mixer
    assert (m.kv_heads, m.vdim, m.rot_dims, m.window, m.rot_scaling) == (2, 8, 8, None, None)
    assert (cfg.embedding_scale, cfg.logit_scale, cfg.logit_softcap, cfg.streams, cfg.loop) == (1.0, 1.0, None, None, None)
    d["layers"][0]["mixer"]["mask"] = None
    d["layers"][0]["mlp"] = None
    cfg = config_from_dict(d)
    assert cfg.layers[0].mixer.window is None and cfg.layers[0].mlp is None


@pytest.mark.parametrize("path,value,match", [
    (("layers", 1, "mixer", "heads"), None, r"layers\[1\]\.mixer\.heads"),
    (("layers", 1, "mixer", "kv_heads"), 3, "multiple"),
    (("layers", 1, "mixer", "rot", "dims"), 7, "even"),
    (("layers", 1, "mixer", "rot", "dims"), 64, "within"),
    (("layers", 1, "mixer", "rot", "scaling", "factor"), 0.0, "positive"),
    (("layers", 1, "mixer", "rot", "scaling", "low"), 9.0, "low < high"),
    (("layers", 1, "mixer", "mask", "size"), 0, "positive"),
    (("layers", 0, "mixer", "tau"), 0.0, "tau"),
    (("layers", 0, "mixer", "dim"), None, r"layers\[0\]\.mixer\.dim"),
    (("layers", 0, "mlp", "kind"), "gated", "not supported"),
    (("layers", 1, "mlp", "router", "top"), 9, "exceeds"),
    (("layers", 1, "mlp", "expert"), None, "expert"),
    (("layers", 0, "type"), "mamba9", "known mixer"),
    (("norm",), None, "norm"),
    (("streams",), 0, "streams"),
    (("streams",), 99, "streams"),
    (("logit_softcap",), -1.0, "logit_softcap"),
    (("loop", "stop"), 9, "loop"),
    (("loop", "times"), 0, "times"),
    (("layers",), [], "non-empty"),
])
def test_bad_configs_name_the_key(path, value, match):
    d = tm.config("A")
    node = d
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ConfigError, match=match):
        config_from_dict(d)


def test_plan_builds_every_layer_from_its_own_entry():
    cfg = config_from_dict(tm.config("A"))
    plan = plan_for(cfg)
    assert [L.mixer.kind for L in plan.layers] == ["gated_linear_attention", "paged_attention", "gated_linear_attention", "paged_attention",
                                                   "gated_linear_attention"]
    assert [L.block.kind for L in plan.layers] == ["hyper"] * 5 and plan.layers[0].block.args["streams"] == 3
    assert [None if L.ffn is None else L.ffn.kind for L in plan.layers] == ["dense_ffn", "moe", "moe", None, "dense_ffn"]
    # the looped span is named once per pass: seven layer runs, each with a cache or state of its own
    assert [e.layer for e in plan.schedule] == [0, 1, 2, 1, 2, 3, 4] and cfg.run_order() == (0, 1, 2, 1, 2, 3, 4)
    a1 = plan.layers[1].mixer.args
    assert (a1["window"], a1["qk_norm_eps"], a1["output_gate"], a1["bias"], a1["scale"], a1["v_head_dim"]) == (20, 1e-5, "elementwise", False, 0.6, 24)
    assert a1["position"].args["scaling"] == {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}
    assert plan.layers[3].mixer.args["position"].args["scaling"] is None
    g = plan.layers[2].mixer.args
    assert (g["n_heads"], g["head_dim"], g["v_head_dim"], g["decay_rank"], g["tau"], g["norm_eps"]) == (3, 8, 16, 4, 3.0, 1e-5)
    e1, e2 = plan.layers[1].ffn.args, plan.layers[2].ffn.args
    assert (e1["n_experts"], e1["top"], e1["ff"], e1["shared_ff"], e1["shared_gate"], e1["router_bias"]) == (8, 2, 24, 40, True, True)
    assert (e2["shared_ff"], e2["shared_gate"], e2["scoring"], e2["renormalize"]) == (0, False, "softmax", True)
    assert (plan.embedding.args["scale"], plan.lm_head.args["scale"], plan.lm_head.args["softcap"]) == (2.0, 1.5, 12.0)
    model = Model(cfg)
    specs = model.param_specs()
    assert {"embed", "final.norm", "head", "l0.mix.a2.b", "l0.mix.norm", "l1.mix.q.norm", "l1.mix.k.norm", "l1.mix.g", "l1.mlp.router.b",
            "l1.mlp.shared.sg", "l1.mlp.e7.down", "l2.mlp.e5.gate", "l3.hc1.mix", "l4.hc2.out", "l4.mlp.up"} <= set(specs)
    assert not any(n.startswith(("l3.mlp", "l3.hc2", "l2.mlp.shared", "l0.mlp.gate")) for n in specs) and "l3.norm2" not in specs
    assert specs["l1.mix.g"].shape == (4 * 24, 64) and specs["l0.mix.a1"].shape == (6, 64) and specs["l0.mix.a2"].shape == (32, 6)
    assert specs["l0.hc1.mix"].shape == (3, 3) and specs["l1.mlp.shared.sg"].shape == (1, 64) and specs["l2.mix.norm"].shape == (16,)
    # cache groups by window, over layer runs: a looped attention layer owns pages once per pass; recurrences own state alone
    mixers = model.schedule_mixers()
    groups, entry_group = plan_groups(plan.schedule, mixers)
    assert [(g.window, g.entries) for g in groups] == [(20, (1, 3)), (33, (5,))]
    assert all(i not in entry_group and mixers[i].cache_spec() is None for i in (0, 2, 4, 6))
    from inferflux_amd.kernels import ops
    assert mixers[2].state_spec().shape == (ops.gla_state_floats(3, 8, 16),) and mixers[2].state_spec().shape[0] >= 3 * 8 * 16
    assert model.graph_safe


def test_one_plain_stream_without_the_key_and_one_stream_with_connections():
    plain = plan_for(config_from_dict(tm.config("C")))
    assert [L.block.kind for L in plain.layers] == ["prenorm"] * 3 and not any("hc1" in n for n in Model(plan=plain).param_specs())
    one = plan_for(config_from_dict(tm.config("B")))
    assert one.layers[0].block.args["streams"] == 1 and Model(plan=one).param_specs()["l0.hc1.mix"].shape == (1, 1)
    assert [e.layer for e in plain.schedule] == [0, 1, 1, 1, 2]


def test_decay_rank_comes_from_the_tensors_where_the_file_leaves_it_out(tmp_path):
    folder = tm.write_model(str(tmp_path / "m"), tm.config("A"), 3)
    import json
    with open(folder + "/config.json") as f:
        assert all("rank" not in L["mixer"] for L in json.load(f)["layers"])
    cfg = load_config(folder)
    assert [L.mixer.rank for L in cfg.layers if L.type == "gla"] == [6, 4, 5]
    bare = tm.config("A")
    for L in bare["layers"]:
        L["mixer"].pop("rank", None)
    with pytest.raises(ConfigError, match="rank"):
        plan_for(config_from_dict(bare))


# ---- the plain implementation's own mechanisms against independent formulas -------------------------------
def test_window_attention_is_a_masked_softmax():
    rng = np.random.default_rng(0)
    T, H, G, d, dv = 9, 4, 2, 6, 5
    q, k, v = rng.normal(size=(T, H, d)), rng.normal(size=(T, G, d)), rng.normal(size=(T, G, dv))
    for size in (None, 1, 3, 9, 40):
        out = pt.window_attention(q, k, v, 0.7, size)
        for h in range(H):
            s = 0.7 * q[:, h] @ k[:, h // 2].T
            i, j = np.arange(T)[:, None], np.arange(T)[None, :]
            seen = (j <= i) & ((i - j < size) if size else True)
            w = np.where(seen, np.exp(s), 0.0)
            assert np.allclose(out[:, h], (w / w.sum(1, keepdims=True)) @ v[:, h // 2])
    assert np.allclose(pt.window_attention(q, k, v, 0.7, 1), np.repeat(v, 2, axis=1))       # a window of one sees itself alone


def test_banded_frequencies_keep_short_waves_slow_long_ones_and_blend_between():
    sc = {"factor": 6.0, "low": 1.0, "high": 3.0, "original": 1024}
    f = pt.banded_frequencies(40, 30000.0, sc)
    base = np.array([30000.0 ** (-2 * i / 40) for i in range(20)])
    assert np.allclose(pt.banded_frequencies(40, 30000.0, None), base)
    wave = 2 * math.pi / base
    kept, slowed = wave < 1024 / 3.0, wave > 1024 / 1.0
    assert kept.any() and slowed.any() and (~kept & ~slowed).any()
    assert np.allclose(f[kept], base[kept]) and np.allclose(f[slowed], base[slowed] / 6.0)
    mid = ~kept & ~slowed
    assert np.all(f[mid] < base[mid]) and np.all(f[mid] > base[mid] / 6.0) and list(f) == sorted(f, reverse=True)
    # at the band's two ends the blend meets its neighbours
    for wl, want in ((1024 / 3.0, 1.0), (1024 / 1.0, 1 / 6.0)):
        s = (1024 / wl - 1.0) / 2.0
        assert np.isclose((1 - s) / 6.0 + s, want)
    x = np.random.default_rng(1).normal(size=(3, 2, 46))
    y = pt.rotate(x, np.array([0, 5, 900]), 40, 30000.0, sc)
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 40:], x[..., 40:])
    assert np.allclose(y[..., :20] ** 2 + y[..., 20:40] ** 2, x[..., :20] ** 2 + x[..., 20:40] ** 2)      # pair (i, i + dims/2) turns
    a = 5 * f[3]
    assert np.allclose(y[1, 0, 3], x[1, 0, 3] * math.cos(a) - x[1, 0, 23] * math.sin(a))
    assert np.allclose(y[1, 0, 23], x[1, 0, 23] * math.cos(a) + x[1, 0, 3] * math.sin(a))


def test_the_recurrence_is_attention_with_decayed_keys_and_carries_on_from_its_state():
    rng = np.random.default_rng(2)
    T, H, d, dv = 19, 2, 5, 3
    q, k, v = rng.normal(size=(T, H, d)), rng.normal(size=(T, H, d)), rng.normal(size=(T, H, dv))
    alpha = rng.uniform(0.3, 1.0, size=(T, H, d))
    o, S = pt.gla_recurrence(q, k, v, alpha)
    # closed form: o_t = sum_{j <= t} (q_t . (k_j * prod_{j < r <= t} alpha_r)) v_j
    for t in (0, 1, 11, 18):
        for h in range(H):
            want = sum(float(q[t, h] @ (k[j, h] * alpha[j + 1:t + 1, h].prod(axis=0))) * v[j, h] for j in range(t + 1))
            assert np.allclose(o[t, h], want)
    o1, S1 = pt.gla_recurrence(q[:7], k[:7], v[:7], alpha[:7])
    o2, S2 = pt.gla_recurrence(q[7:], k[7:], v[7:], alpha[7:], S1)
    assert np.allclose(np.concatenate([o1, o2]), o) and np.allclose(S2, S)
    W = {"x.a1": rng.normal(size=(3, 8)), "x.a2": rng.normal(size=(10, 3)), "x.a2.b": rng.normal(size=10)}
    h = rng.normal(size=(4, 8))
    al = pt.gla_decay(h, W, "x.", 16.0)
    assert np.all((al > 0) & (al < 1)) and np.allclose(al ** 16.0, 1 / (1 + np.exp(-((h @ W["x.a1"].T) @ W["x.a2"].T + W["x.a2.b"]))))


def test_router_takes_the_largest_biased_logits_and_a_softmax_over_them():
    rng = np.random.default_rng(3)
    W = {"r.router": rng.normal(size=(6, 4)), "r.router.b": np.array([0.0, 0.0, 50.0, 0.0, 0.0, -50.0])}
    h = rng.normal(size=(5, 4))
    ids, w = pt.route(h, W, "r.", 3)
    z = h @ W["r.router"].T + W["r.router.b"]
    assert np.all(ids[:, 0] == 2) and not np.any(ids == 5) and np.allclose(w.sum(1), 1.0) and np.all(w[:, 0] > 0.99)
    for t in range(5):
        assert set(ids[t]) == set(np.argsort(-z[t])[:3])
        assert np.allclose(w[t], np.exp(z[t, ids[t]]) / np.exp(z[t, ids[t]]).sum())
    one, w1 = pt.route(h, W, "r.", 1)
    assert np.allclose(w1, 1.0)


def test_hyper_connections_with_an_identity_are_the_ordinary_residual():
    rng = np.random.default_rng(4)
    S, T, H = 3, 5, 7
    xs = rng.normal(size=(S, T, H))
    sub = lambda u: np.tanh(u) * 2.0
    W = {"h.in": np.array([1.0, 0.0, 0.0]), "h.out": np.array([1.0, 0.0, 0.0]), "h.mix": np.eye(3)}
    out = pt.hyper_step(xs, W, "h.", sub)
    assert np.allclose(out[0], xs[0] + sub(xs[0])) and np.allclose(out[1:], xs[1:])
    W = {"h.in": rng.normal(size=3), "h.out": rng.normal(size=3), "h.mix": rng.normal(size=(3, 3))}
    out = pt.hyper_step(xs, W, "h.", sub)
    y = sub(sum(W["h.in"][s] * xs[s] for s in range(S)))
    for t in range(S):          # the matrix is indexed [from, to]
        assert np.allclose(out[t], sum(W["h.mix"][s, t] * xs[s] for s in range(S)) + W["h.out"][t] * y)


def test_activations_and_norm():
    z = np.linspace(-5, 5, 101)
    from math import erf
    exact = np.array([0.5 * x * (1 + erf(x / math.sqrt(2))) for x in z])
    assert np.abs(pt.gelu_tanh(z) - exact).max() < 1e-3 and pt.gelu_tanh(np.array([0.0]))[0] == 0.0
    assert np.allclose(pt.silu(z), z / (1 + np.exp(-z)))
    x = np.random.default_rng(5).normal(size=(3, 11))
    assert np.allclose(pt.rms_norm(x, np.ones(11), 0.0) ** 2 @ np.ones(11), 11.0)
    assert np.allclose(pt.rms_norm(np.zeros((1, 4)), np.ones(4), 1e-6), 0.0)               # eps sits inside the root
    assert np.allclose(pt.rms_norm(x * 1e-4, np.ones(11), 1.0), x * 1e-4, rtol=1e-6)


def test_the_whole_model_changes_when_a_mechanism_is_left_out(tmp_path):
    """What the engine's tests rely on: every mechanism moves the plain model's logits by far more than rounding."""
    folder = tm.write_model(str(tmp_path / "m"), tm.config("A"), 5, gain=2.0, keep_rank=True)
    cfg, W = tm.load_plain(folder)
    ids = list(np.random.default_rng(3).integers(0, 300, size=60))
    base = pt.forward(cfg, W, ids)
    scale = np.abs(base).max()

    def changed(edit=None, weights=None):
        c2 = tm.config("A")
        if edit:
            edit(c2)
        return np.abs(pt.forward(c2, weights or W, ids) - base).max() / scale

    assert changed() == 0.0
    assert changed(lambda c: c["layers"][1]["mixer"]["mask"].update(size=21)) > 1e-3
    assert changed(lambda c: c["layers"][3]["mixer"]["mask"].update(size=32)) > 1e-3
    assert changed(lambda c: c["layers"][1]["mixer"]["rot"].pop("scaling")) > 1e-3
    assert changed(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6)) > 1e-3
    assert changed(lambda c: c["layers"][0]["mixer"].update(tau=7.0)) > 1e-3
    assert changed(lambda c: c["layers"][1]["mlp"]["router"].update(top=3)) > 1e-3
    assert changed(lambda c: c["layers"][1]["mlp"].pop("shared")) > 1e-3
    assert changed(lambda c: c["loop"].update(times=1)) > 1e-3
    assert changed(lambda c: c.update(logit_softcap=11.0)) > 1e-3
    assert changed(lambda c: c.update(logit_scale=1.4)) > 1e-3
    assert changed(lambda c: c["embedding"].update(scale=2.1)) > 1e-3
    for name, edit in (("l0.mix.a2.b", lambda t: t + 0.5), ("l1.mlp.router.b", lambda t: t[::-1].copy()), ("l1.mix.q.norm", lambda t: t * 0 + 1.0),
                       ("l2.hc1.mix", lambda t: t.T.copy()), ("l1.mlp.shared.sg", lambda t: -t), ("l2.mix.norm", lambda t: t * 0 + 1.0),
                       ("l3.hc1.in", lambda t: t[::-1].copy())):
        W2 = dict(W)
        W2[name] = edit(W[name])
        assert changed(weights=W2) > 1e-3, name


def test_random_weights_folder_roundtrips(tmp_path):
    """The seeded random-weights mode writes every tensor the plan declares, decays' biases in the range a recurrence needs."""
    import torch
    from safetensors.torch import load_file
    from inferflux_amd.weights import write_random_model
    cfg = config_from_dict(tm.config("D"))
    folder = str(tmp_path / "m")
    write_random_model(folder, cfg, seed=3)
    assert load_config(folder) == cfg
    t = load_file(folder + "/model.safetensors")
    assert set(t) == set(Model(cfg).param_specs())
    assert float(t["l0.mix.a2.b"].float().min()) >= 0.0 and t["l0.hc1.mix"].shape == (5, 5)
    logits = pt.forward(tm.config("D"), {k: v.double().numpy() for k, v in t.items()}, [1, 2, 3, 4])
    assert np.isfinite(logits).all() and np.abs(logits).max() <= 8.0
