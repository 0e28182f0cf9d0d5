"""Givozen on the CPU: the plain implementation's functions against cases with known answers, the configuration reader's
refusals, and the assembly's tensor list and run order."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest

import plain_givozen as plain
from givozen_cases import CONFIGS, CONFIG_A, CONFIG_C, CONFIG_D, model_folder, load_plain, routed_runs


def test_offset_norm_has_unit_gain_at_a_zero_weight_and_eps_inside_the_root():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 17)) * 5
    y = plain.offset_norm(x, np.zeros(17), 0.0)
    assert np.allclose((y * y).mean(-1), 1.0)
    w = rng.normal(size=17) * 0.1
    assert np.allclose(plain.offset_norm(x, w, 3.0), x / np.sqrt((x * x).mean(-1, keepdims=True) + 3.0) * (1.0 + w))


def test_frequencies_rescaled_by_wavelength():
    f = plain.wavelength_scaled_frequencies(8, 10000.0, None)
    assert np.allclose(f, 10000.0 ** (-np.arange(4) / 4.0))
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    g = plain.wavelength_scaled_frequencies(8, 10000.0, sc)
    wavelength = 2 * math.pi / f
    # pair 0 (wavelength 6.3 < 16) keeps its frequency, pairs 2 and 3 (628 and 6283 > 64) turn four times slower
    assert wavelength[0] < 16 and g[0] == f[0]
    assert wavelength[2] > 64 and np.allclose(g[2:], f[2:] / 4.0)
    # pair 1 (wavelength 62.8) lies between: s = (64 / 62.8 - 1) / 3
    s = (64 / wavelength[1] - 1.0) / 3.0
    assert 16 < wavelength[1] < 64 and np.isclose(g[1], (1 - s) * f[1] / 4.0 + s * f[1])
    # other constants move the borders: with low 0.01 no wavelength is long enough to be slowed down fully
    h = plain.wavelength_scaled_frequencies(8, 10000.0, {"factor": 4.0, "low": 0.01, "high": 4.0, "original": 64})
    assert np.all(h[1:] > f[1:] / 4.0) and h[0] == f[0]


def test_rotation_in_halves_keeps_lengths_and_depends_on_distance():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(5, 2, 12))
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    y = plain.rotate_halves(x, [0, 1, 7, 100, 1000], 8, 10000.0, sc)
    assert np.allclose(y[..., 8:], x[..., 8:]) and np.allclose(y[0], x[0])
    assert np.allclose(np.linalg.norm(y[..., :8], axis=-1), np.linalg.norm(x[..., :8], axis=-1))
    # dim i turns with dim i + dims/2: a vector with only dims 1 and 5 set stays in those two
    e = np.zeros((1, 1, 12))
    e[0, 0, 1], e[0, 0, 5] = 1.0, 2.0
    r = plain.rotate_halves(e, [3], 8, 10000.0, None)[0, 0]
    a = 3 * 10000.0 ** (-2 / 8)
    assert np.allclose(r[[1, 5]], [math.cos(a) - 2 * math.sin(a), 2 * math.cos(a) + math.sin(a)]) and np.count_nonzero(r) == 2
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    at = lambda v, p: plain.rotate_halves(v, [p], 8, 500.0, sc)[0, 0]
    assert np.isclose(at(q, 9) @ at(k, 4), at(q, 105) @ at(k, 100))


def test_attention_is_causal_groups_heads_and_takes_a_temperature_a_head():
    rng = np.random.default_rng(2)
    T, H, G, D, V = 7, 4, 2, 5, 3
    q, k, v = rng.normal(size=(T, H, D)), rng.normal(size=(T, G, D)), rng.normal(size=(T, G, V))
    temp = np.array([1.0, 0.0, 2.0, 0.5])
    o = plain.causal_attention(q, k, v, 0.3, temp)
    assert np.allclose(o[0, 0], v[0, 0]) and np.allclose(o[0, 3], v[0, 1])          # the first row sees itself only
    assert np.allclose(o[4, 1], v[:5, 0].mean(0))                                    # temperature 0: the mean of the visible values
    s = q[5, 2] @ k[:6, 1].T * 0.3 * 2.0
    p = np.exp(s - s.max())
    assert np.allclose(o[5, 2], (p / p.sum()) @ v[:6, 1])
    # a later row changes nothing before it
    k2, v2 = k.copy(), v.copy()
    k2[6], v2[6] = 9.0, -9.0
    assert np.allclose(plain.causal_attention(q, k2, v2, 0.3, temp)[:6], o[:6])


def test_attention_mixer_biases_gate_and_output():
    rng = np.random.default_rng(3)
    T, E, H, G, D, V = 4, 6, 2, 1, 4, 3
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.5, "rot": {"base": 100.0, "dims": 0}}
    w = {"p.q": np.zeros((H * D, E)), "p.q.b": np.zeros(H * D), "p.k": np.zeros((G * D, E)), "p.k.b": np.zeros(G * D),
         "p.v": rng.normal(size=(G * V, E)), "p.v.b": rng.normal(size=G * V), "p.temp": np.ones(H), "p.g": rng.normal(size=(H, E)),
         "p.o": np.eye(H * V)}
    h = rng.normal(size=(T, E))
    out = plain.attention_mixer(h, w, "p.", m, np.arange(T))
    # all scores equal: each row is the running mean of the biased values, times the row's own gate a head
    values = h @ w["p.v"].T + w["p.v.b"]
    mean = np.cumsum(values, axis=0) / np.arange(1, T + 1)[:, None]
    gate = plain.sigmoid(h @ w["p.g"].T)
    assert np.allclose(out, np.concatenate([mean * gate[:, :1], mean * gate[:, 1:]], axis=1))


def test_polynomial_of_unit_rms_powers():
    rng = np.random.default_rng(4)
    z = rng.normal(size=(3, 11))
    assert np.allclose(plain.poly_norm(z, [1, 0, 0, 0], 0.0), z / np.sqrt((z * z).mean(-1, keepdims=True)))
    assert np.allclose(plain.poly_norm(z, [0, 0, 0, 0.25], 1e-6), 0.25)
    full = plain.poly_norm(z, [0.5, -2.0, 3.0, 0.1], 1e-3)
    want = sum(c * (z ** p) / np.sqrt((z ** (2 * p)).mean(-1, keepdims=True) + 1e-3) for c, p in ((0.5, 1), (-2.0, 2), (3.0, 3))) + 0.1
    assert np.allclose(full, want)
    # each power is normed by itself: scaling z changes nothing when eps is 0
    assert np.allclose(plain.poly_norm(7.0 * z, [0.5, -2.0, 3.0, 0.1], 0.0), plain.poly_norm(z, [0.5, -2.0, 3.0, 0.1], 0.0))


def test_clamped_gated_expert():
    w = {"e.gate": np.array([[1.0, 0.0]]), "e.up": np.array([[0.0, 1.0]]), "e.down": np.array([[1.0]])}
    f = lambda g, u, limit=2.0: float(plain.clamped_glu_expert(np.array([[g, u]]), w, "e.", limit)[0, 0])
    assert np.isclose(f(0.5, 0.25), 0.5 * plain.sigmoid(1.702 * 0.5) * 1.25)
    assert np.isclose(f(9.0, 0.25), 2.0 * plain.sigmoid(1.702 * 2.0) * 1.25)            # the gate is clamped from above only
    assert np.isclose(f(-9.0, 0.25), -9.0 * plain.sigmoid(1.702 * -9.0) * 1.25)
    assert np.isclose(f(0.5, 9.0), 0.5 * plain.sigmoid(0.851) * 3.0) and np.isclose(f(0.5, -9.0), 0.5 * plain.sigmoid(0.851) * -1.0)
    assert np.isclose(f(0.5, 9.0, limit=0.3), 0.3 * plain.sigmoid(1.702 * 0.3) * 1.3)


def test_router_weights_multiply_the_experts_input():
    rng = np.random.default_rng(5)
    T, E, F, X = 5, 6, 4, 4
    w = {"m.router": rng.normal(size=(X, E))}
    for e in range(X):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = rng.normal(size=(F, E)), rng.normal(size=(F, E)), rng.normal(size=(E, F))
    mlp = {"expert": {"ff": F, "limit": 1.0}, "router": {"experts": X, "top": 2}}
    h = rng.normal(size=(T, E))
    ids, scores, all_scores = plain.route(h, w["m.router"], 2)
    z = h @ w["m.router"].T
    for t in range(T):
        assert list(ids[t]) == sorted(range(X), key=lambda e: (-z[t, e], e))[:2]
    assert np.allclose(scores, plain.sigmoid(np.take_along_axis(z, ids, 1)))          # not renormalized
    out = plain.moe_ff(h, w, "m.", mlp)
    want = np.stack([sum(plain.clamped_glu_expert(scores[t, j] * h[t:t + 1], w, f"m.e{ids[t, j]}.", 1.0)[0] for j in range(2)) for t in range(T)])
    assert np.allclose(out, want)
    # the unit is not linear, so the weight on the input is not the weight on the output
    other = np.stack([sum(scores[t, j] * plain.clamped_glu_expert(h[t:t + 1], w, f"m.e{ids[t, j]}.", 1.0)[0] for j in range(2)) for t in range(T)])
    assert not np.allclose(out, other)
    # handed picks replace the router's choice, the scores stay the router's
    forced = np.array([[3, 0]] * T)
    got = plain.moe_ff(h, w, "m.", mlp, picks=forced)
    assert np.allclose(got[0], sum(plain.clamped_glu_expert(all_scores[0, e] * h[:1], w, f"m.e{e}.", 1.0)[0] for e in (3, 0)))
    # a shared expert runs for every row behind its own switch
    w["m.shared.gate"], w["m.shared.up"], w["m.shared.down"] = rng.normal(size=(3, E)), rng.normal(size=(3, E)), rng.normal(size=(E, 3))
    w["m.shared.sg"] = rng.normal(size=(1, E))
    with_shared = plain.moe_ff(h, w, "m.", dict(mlp, shared={"ff": 3, "limit": 0.4}))
    assert np.allclose(with_shared - out, plain.sigmoid(h @ w["m.shared.sg"].T) * plain.clamped_glu_expert(h, w, "m.shared.", 0.4))


def test_run_order_of_a_repeated_run_of_layers():
    assert plain.run_order({"layers": [0] * 3}) == [(0, None, False), (1, None, False), (2, None, False)]
    assert plain.run_order(CONFIG_A) == [(0, None, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (1, 2, True), (2, 2, False),
                                         (3, None, False)]
    assert plain.run_order(CONFIG_D) == [(0, None, False), (1, 0, True)]
    assert routed_runs(CONFIG_A) == [1, 2, 3, 4, 5, 6] and routed_runs(CONFIG_C) == [0, 2]


def test_pass_vectors_and_the_embedding_rows_enter_before_each_pass():
    config, w = load_plain(model_folder("C"))
    tokens = [5, 9, 77, 3]
    base = plain.forward(config, w, tokens)
    # the second pass's vector matters, and so does the embedding added before it: without both, the logits are others
    w2 = dict(w)
    w2["loop.step"] = w["loop.step"].copy()
    w2["loop.step"][1] += 0.5
    assert np.abs(plain.forward(config, w2, tokens) - base).max() > 1e-3
    # one pass instead of two is another model
    assert np.abs(plain.forward(dict(config, loop={"start": 0, "stop": 2, "times": 1}), w, tokens) - base).max() > 1e-3
    # by hand for the first layer run: x = embed + step[0], then the layer
    _, layers = plain.forward(config, w, tokens, keep_layers=True)
    x = w["embed"][tokens] + w["loop.step"][0]
    y = plain.attention_mixer(plain.offset_norm(x, w["l0.norm1"], 1e-6), w, "l0.mix.", config["layers"][0]["mixer"], np.arange(4))
    x = x + plain.offset_norm(y, w["l0.norm1b"], 1e-6)
    x = x + plain.offset_norm(plain.moe_ff(plain.offset_norm(x, w["l0.norm2"], 1e-6), w, "l0.mlp.", config["layers"][0]["mlp"]), w["l0.norm2b"], 1e-6)
    assert np.allclose(layers[0], x) and layers.shape[0] == 4


# ---------------------------------------------------------------------------- configuration and assembly
def test_configuration_round_trip_and_refusals():
    from llmx_amd.config import ConfigError
    from llmx_amd.models import read_config
    for name, config in CONFIGS.items():
        cfg = read_config(copy.deepcopy(config))
        assert cfg.architecture == "Givozen" and read_config(cfg.to_json()) == cfg, name

    def refused(edit, text):
        c = copy.deepcopy(CONFIG_A)
        edit(c)
        with pytest.raises(ConfigError) as e:
            read_config(c)
        assert text in str(e.value), str(e.value)

    refused(lambda c: c["layers"][1]["mixer"].pop("scale"), "missing key layers[1].mixer.scale")
    refused(lambda c: c["layers"][0]["mixer"].update(window=5), "layers[0].mixer.window is not one this engine reads")
    refused(lambda c: c["layers"][0].update(type="gla"), "layers[0].type")
    refused(lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "layers[1].mlp.router.top")
    refused(lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "missing key layers[1].mlp.expert.limit")
    refused(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "layers[0].mixer.rot.dims")
    refused(lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "layers[0].mixer.kv_heads")
    refused(lambda c: c["loop"].update(stop=9), "loop")
    refused(lambda c: c["loop"].update(times=0), "loop.times")
    refused(lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].update(high=0.5), "rot.scaling.high")
    refused(lambda c: c.update(softcap=3.0), "key softcap is not one this engine reads")
    # a model without a loop and a rotation without scaling are configurations of the design
    c = copy.deepcopy(CONFIG_A)
    del c["loop"]
    del c["layers"][0]["mixer"]["rot"]["scaling"]
    assert read_config(c).loop is None


def test_assembly_lists_the_tensors_and_the_run_order():
    from llmx_amd.models import read_config, registry
    from llmx_amd.weights.folder import model_tensor_specs
    cfg = read_config(copy.deepcopy(CONFIG_A))
    spec = registry.assemble(cfg)
    assert [(e.layer, e.cache, e.before) for e in spec.run_order] == [(0, 0, None), (1, 1, 0), (2, 2, None), (1, 3, 1), (2, 4, None), (1, 5, 2),
                                                                      (2, 6, None), (3, 7, None)]
    assert [p.params["add_embedding"] for p in spec.inputs] == [False, True, True]
    names = {s.name: s for s in model_tensor_specs(cfg)}
    want = {"embed", "loop.step", "final.norm"}
    for i, layer in enumerate(CONFIG_A["layers"]):
        want |= {f"l{i}.norm1", f"l{i}.norm1b"} | {f"l{i}.mix.{t}" for t in ("q", "q.b", "k", "k.b", "v", "v.b", "temp", "g", "o")}
        mlp = layer["mlp"]
        if mlp:
            want |= {f"l{i}.norm2", f"l{i}.norm2b"}
            if mlp["kind"] == "dense":
                want |= {f"l{i}.mlp.{t}" for t in ("up", "down", "act")}
            else:
                want |= {f"l{i}.mlp.router"} | {f"l{i}.mlp.e{e}.{t}" for e in range(mlp["router"]["experts"]) for t in ("gate", "up", "down")}
                if "shared" in mlp:
                    want |= {f"l{i}.mlp.shared.{t}" for t in ("gate", "up", "down", "sg")}
    assert set(names) == want
    assert names["loop.step"].shape == (3, 128) and names["l1.mix.g"].shape == (8, 128) and names["l1.mix.temp"].shape == (8,)
    assert names["l0.mlp.act"].shape == (4,) and names["l1.mlp.shared.sg"].shape == (1, 128) and names["l2.mix.q"].shape == (128, 128)
    # a configuration without a loop has no pass vectors
    c = copy.deepcopy(CONFIG_A)
    del c["loop"]
    assert "loop.step" not in {s.name for s in model_tensor_specs(read_config(c))}
    # the rotary table of the rescaled frequencies is the plain function's
    from llmx_amd.parts.position import scaled_table
    sc = {"factor": 8.0, "low": 2.0, "high": 16.0, "original": 32}
    table = scaled_table(50, 16, 5000.0, sc)
    f = plain.wavelength_scaled_frequencies(16, 5000.0, sc)
    angle = np.arange(50)[:, None] * f[None, :]
    assert np.allclose(table[:, :8], np.cos(angle), atol=1e-7) and np.allclose(table[:, 8:], np.sin(angle), atol=1e-7)
