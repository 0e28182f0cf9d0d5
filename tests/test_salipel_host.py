"""Salipel on the CPU: pins of the plain implementation (tests/plain_salipel.py), the configuration reader's round trip and
refusals, the assembly's tensor list and cache needs, and the cache manager's kept first pages and chunked release."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest

import plain_salipel as plain
from salipel_cases import CONFIGS, CONFIG_A, CONFIG_B, CONFIG_C


# ---------------------------------------------------------------------------- the plain implementation's pins
def test_masks_say_who_sees_whom():
    m = plain.mask_window_keep_first(12, 4, 2)
    assert m[11].tolist() == [True, True] + [False] * 6 + [True] * 4      # keys 0, 1 kept; 8..11 in the window
    assert m[3].tolist() == [True] * 4 + [False] * 8
    assert not plain.mask_window_keep_first(12, 4, 0)[11, 7] and plain.mask_window_keep_first(12, 4, 0)[11, 8]
    c = plain.mask_chunks(10, 4)
    assert c[7].tolist() == [False] * 4 + [True] * 4 + [False] * 2 and c[8].tolist() == [False] * 8 + [True, False]
    assert plain.mask_causal(3).tolist() == [[True, False, False], [True, True, False], [True, True, True]]


def test_a_sink_only_takes_weight_and_a_far_sink_takes_none():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(5, 2, 4)), rng.normal(size=(5, 1, 4)), rng.normal(size=(5, 1, 3))
    mask = plain.mask_causal(5)
    bare = plain.masked_softmax_attention(q, k, v, 0.5, mask)
    assert np.allclose(plain.masked_softmax_attention(q, k, v, 0.5, mask, sink=np.array([-80.0, -80.0])), bare)
    sunk = plain.masked_softmax_attention(q, k, v, 0.5, mask, sink=np.array([0.0, 50.0]))
    s0 = q[0, 0] @ k[0, 0] * 0.5          # the first row sees one key: its weight is e^s / (e^s + e^sink)
    assert np.allclose(sunk[0, 0], v[0, 0] * math.exp(s0) / (math.exp(s0) + 1.0))
    assert np.abs(sunk[:, 1]).max() < 1e-15


def test_distance_slopes_and_their_sign():
    s = plain.distance_slopes(8)
    assert np.allclose(s, [2.0 ** -(a + 1) for a in range(8)]) and np.allclose(plain.distance_slopes(2), [2.0 ** -4, 2.0 ** -8])
    # the nearer of two equal keys gets the larger weight
    q, k = np.ones((3, 1, 2)), np.ones((3, 1, 2))
    v = np.eye(3)[:, None, :]
    i, j = np.arange(3)[:, None], np.arange(3)[None, :]
    o = plain.masked_softmax_attention(q, k, v, 1.0, plain.mask_causal(3), bias=np.array([0.5])[:, None, None] * (i - j)[None])
    assert o[2, 0, 2] > o[2, 0, 1] > o[2, 0, 0] and np.isclose(o[2, 0, 1] / o[2, 0, 2], math.exp(-0.5))


def test_rescaled_frequencies_three_ranges_and_rotation():
    f = plain.wavelength_scaled_frequencies(16, 10000.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64})
    bare = plain.wavelength_scaled_frequencies(16, 10000.0, None)
    wl = 2 * math.pi / bare
    assert np.allclose(f[wl < 16], bare[wl < 16]) and np.allclose(f[wl > 64], bare[wl > 64] / 4.0)
    mid = (wl >= 16) & (wl <= 64)
    assert mid.any() and np.all(f[mid] < bare[mid]) and np.all(f[mid] > bare[mid] / 4.0)
    x = np.random.default_rng(1).normal(size=(6, 2, 8))
    r = plain.rotate_halves(x, np.arange(6), {"base": 100.0, "dims": 4})
    assert np.allclose(r[..., 4:], x[..., 4:]) and np.allclose(r[0], x[0])
    assert np.allclose(np.hypot(r[..., 0], r[..., 2]), np.hypot(x[..., 0], x[..., 2]))     # dims 0 and 2 are a pair
    # relative positions: scores of rotated vectors depend on the distance only
    a = plain.rotate_halves(np.tile(x[:1], (6, 1, 1)), np.arange(6), {"base": 100.0, "dims": 8})
    assert np.isclose(a[1, 0] @ a[3, 0], a[2, 0] @ a[4, 0])


def _memory_weights(rng, E, H, D, V, gate_scale=1.0):
    W = {"m." + n: rng.normal(size=s) * 0.4 for n, s in (("q", (H * D, E)), ("k", (H * D, E)), ("v", (H * V, E)), ("g", (H * V, E)),
                                                         ("o", (E, H * V)), ("i", (H, E)), ("f", (H, E)))}
    W["m.i"] *= gate_scale
    W["m.f"] *= gate_scale
    W.update({"m.i.b": rng.normal(size=H), "m.f.b": rng.normal(size=H) + 2.0, "m.norm": rng.uniform(0.5, 1.5, size=H * V)})
    return W


def test_matrix_memory_against_the_sums_written_out_and_across_a_cut():
    rng = np.random.default_rng(2)
    E, H, D, V, T = 12, 2, 5, 3, 9
    cfg = {"heads": H, "dim": D, "vdim": V, "gate_cap": 6.0}
    W = _memory_weights(rng, E, H, D, V, 3.0)
    h = rng.normal(size=(T, E))
    y, state = plain.matrix_memory(h, W, "m.", cfg, 1e-6)
    # cut in two: the state carries everything
    y1, s1 = plain.matrix_memory(h[:4], W, "m.", cfg, 1e-6)
    y2, s2 = plain.matrix_memory(h[4:], W, "m.", cfg, 1e-6, state=s1)
    assert np.allclose(np.concatenate([y1, y2]), y, atol=1e-12) and all(np.allclose(a, b) for a, b in zip(s2, state))
    # the same read-out from the sums written out, without a running maximum: weights exp(i_j + sum of later f)
    cap = 6.0
    gi = cap * np.tanh((h @ W["m.i"].T + W["m.i.b"]) / cap)
    gf = np.log(plain.sigmoid(cap * np.tanh((h @ W["m.f"].T + W["m.f.b"]) / cap)))
    t, a = T - 1, 1
    q = (W["m.q"] @ h[t]).reshape(H, D)[a] * D ** -0.5
    logw = np.array([gi[j, a] + gf[j + 1:t + 1, a].sum() for j in range(t + 1)])
    ks = np.stack([(W["m.k"] @ h[j]).reshape(H, D)[a] for j in range(t + 1)])
    vs = np.stack([(W["m.v"] @ h[j]).reshape(H, V)[a] for j in range(t + 1)])
    num = (np.exp(logw)[:, None] * (ks @ q)[:, None] * vs).sum(0)
    den_n = (np.exp(logw) * (ks @ q)).sum()
    m_t = state[2][a]
    want = num * math.exp(-m_t) / (max(abs(den_n) * math.exp(-m_t), math.exp(-m_t)) + 1e-6)
    S, n, _ = state
    got = (S[a].T @ q) / (max(abs(n[a] @ q), math.exp(-m_t)) + 1e-6)
    assert np.allclose(got, want)
    # the running maximum starts at 0, not at minus infinity: with very negative input gates it stays at f's running sum or above i
    low = dict(W)
    low["m.i.b"] = np.full(H, -50.0)
    _, (_, _, m_low) = plain.matrix_memory(h[:1], low, "m.", cfg, 1e-6)
    assert np.all(m_low > -1.0)          # max(f + 0, i) with f = log sigmoid(.) > -6.1 and here close to 0; never i = -6


def test_two_maps_difference_lambda_and_norm():
    rng = np.random.default_rng(3)
    E, H, G, D, V, T = 10, 2, 1, 4, 6, 7
    cfg = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.5, "softcap": 2.0, "diff": 0.4, "rot": {"base": 50.0, "dims": 4}}
    W = {"a." + n: rng.normal(size=s) * 0.5 for n, s in (("q", (H * 2 * D, E)), ("k", (G * 2 * D, E)), ("v", (G * V, E)), ("g", (H * V, E)),
                                                         ("lq1", (D,)), ("lk1", (D,)), ("lq2", (D,)), ("lk2", (D,)))}
    W.update({"a.q.norm": rng.uniform(0.5, 1.5, size=D), "a.k.norm": rng.uniform(0.5, 1.5, size=D), "a.o": np.eye(H * V)})
    lam = plain.difference_lambda(W, "a.", 0.4)
    assert np.isclose(lam, math.exp(W["a.lq1"] @ W["a.lk1"]) - math.exp(W["a.lq2"] @ W["a.lk2"]) + 0.4)
    h = rng.normal(size=(T, E))
    y = plain.difference_attention(h, W, "a.", cfg, 1e-6)
    # before the gate every head has root mean square 1 - diff (a little less where eps counts beside a small difference)
    bare = y / plain.sigmoid(h @ W["a.g"].T)
    assert np.allclose(np.sqrt((bare.reshape(T, H, V) ** 2).mean(-1)), 0.6, atol=3e-4)
    # the first row sees one key in both maps: a1 = a2 = v, so its direction is v's (or its opposite)
    v0 = (W["a.v"] @ h[0]).reshape(G, V)[0]
    first = bare[0].reshape(H, V)[0]
    assert np.allclose(np.abs(first) / np.linalg.norm(first), np.abs(v0) / np.linalg.norm(v0), atol=1e-4)
    # map 2 uses the second half of a head's q and k rows: zeroing them makes its scores 0, i.e. a plain average of the values
    Wz = dict(W)
    Wz["a.q"] = W["a.q"].copy()
    Wz["a.q"].reshape(H, 2, D, E)[:, 1] = 0.0
    assert not np.allclose(plain.difference_attention(h, Wz, "a.", cfg, 1e-6), y)


def test_routing_scores_choice_and_weights():
    rng = np.random.default_rng(4)
    E, X = 6, 5
    W = {"r.router": rng.normal(size=(X, E)), "r.correction": np.array([0.0, 0.0, 5.0, 0.0, 0.0])}
    cfg = {"router": {"experts": X, "top": 2, "scale": 3.0}}
    h = rng.normal(size=(8, E))
    ids, w, z = plain.route(h, W, "r.", cfg)
    s = plain.softmax_rows(z)
    assert np.all(ids[:, 0] == 2)                          # the correction decides the choice ...
    assert np.allclose(w.sum(-1), 3.0)                     # ... the weights are normalized, then scaled ...
    assert np.allclose(w[:, 0] / w[:, 1], s[np.arange(8), 2] / s[np.arange(8), ids[:, 1]])     # ... and come from the scores alone
    W["r.correction"] = np.zeros(X)
    z2 = np.tile(np.array([[1.0, 2.0, 2.0, 0.0, 2.0]]), (1, 1))
    W["r.router"] = np.linalg.lstsq(h[:1].T @ h[:1] + np.eye(E) * 1e-9, h[:1].T @ z2, rcond=None)[0].T
    assert plain.route(h[:1], W, "r.", cfg)[0].tolist() in ([[1, 2]], [[1, 4]], [[2, 4]])


def test_units():
    z = np.array([-2.0, -0.1, 0.0, 0.3, 3.0])
    assert np.allclose(plain.gelu_tanh(z), 0.5 * z * (1 + np.tanh(0.7978845608 * (z + 0.044715 * z ** 3))))
    W = {"e.router": np.zeros((1, 2)), "e.correction": np.zeros(1), "e.e0.up": np.array([[1.0, 0.0], [0.0, -1.0]]), "e.e0.down": np.eye(2)}
    out = plain.routed_units(np.array([[2.0, 3.0]]), W, "e.", {"router": {"experts": 1, "top": 1, "scale": 1.0}})
    assert np.allclose(out, [[4.0, 0.0]])                  # the square of relu; one pick weighs scale


def test_a_layer_is_one_norm_and_a_constant_on_the_sum():
    from salipel_cases import plain as plain_of
    config, W = plain_of("B")
    x = np.random.default_rng(5).normal(size=(6, config["width"]))
    i = 1
    entry, eps = config["layers"][i], config["norm"]["eps"]
    h = plain.rms_norm(x, W[f"l{i}.norm1"], eps)
    want = x + config["residual_mult"] * (plain.side_by_side(h, W, f"l{i}.mix.", entry["mixer"], eps) + plain.dense_unit(h, W, f"l{i}.mlp."))
    assert np.allclose(plain.layer(x, W, i, config), want)


# ---------------------------------------------------------------------------- configuration and assembly
def test_configuration_round_trip_and_refusals():
    from llmx_amd.config import ConfigError
    from llmx_amd.models import read_config
    for name, config in CONFIGS.items():
        cfg = read_config(copy.deepcopy(config))
        again = read_config(cfg.to_json())
        assert again == cfg and cfg.vocab_size == config["vocab"], name
    assert read_config(copy.deepcopy(CONFIG_B)).layers[1].mixer.left.keep_first == 0      # not stated: none kept

    def refused(edit, text):
        c = copy.deepcopy(CONFIG_A)
        edit(c)
        with pytest.raises(ConfigError, match=text):
            read_config(c)

    refused(lambda c: c["layers"][1]["mixer"]["left"].pop("scale"), r"missing key layers\[1\]\.mixer\.left\.scale")
    refused(lambda c: c["layers"][0]["mixer"].update(window=3), r"layers\[0\]\.mixer\.window is not one this engine reads")
    refused(lambda c: c["layers"][2].update(type="attention_3"), r"layers\[2\]\.type")
    refused(lambda c: c["layers"][1]["mlp"]["router"].update(top=9), r"layers\[1\]\.mlp\.router\.top")
    refused(lambda c: c["layers"][1]["mixer"]["left"].update(vdim=48), r"layers\[1\]\.mixer\.left\.vdim")
    refused(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), r"layers\[0\]\.mixer\.rot\.dims")
    refused(lambda c: c.pop("residual_mult"), "missing key residual_mult")
    refused(lambda c: c["layers"][1]["mixer"]["right"].update(gate_cap=0.0), r"layers\[1\]\.mixer\.right\.gate_cap")
    refused(lambda c: c.update(loop={"start": 0}), "key loop is not one this engine reads")


def test_assembly_lists_the_designs_tensors_and_cache_needs():
    import torch
    from llmx_amd.engine.model import BuiltModel
    from llmx_amd.models import read_config, registry
    from llmx_amd.parts.base import BuildContext
    from llmx_amd.parts.spec import CompositeNeed, PagedNeed, StateNeed
    cfg = read_config(copy.deepcopy(CONFIG_A))
    model = BuiltModel(registry.assemble(cfg), BuildContext(torch.float32, torch.device("cpu"), 64, 16))
    names = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert names["l0.mix.q"] == (4 * 2 * 32, 128) and names["l0.mix.k"] == (2 * 2 * 32, 128) and names["l0.mix.v"] == (2 * 64, 128)
    assert names["l0.mix.lq1"] == (32,) and names["l0.mix.g"] == (4 * 64, 128) and names["l0.mix.q.norm"] == (32,)
    assert "l1.mix.left.v" not in names and names["l1.mix.left.g"] == (4 * 32, 128) and names["l1.mix.right.norm"] == (2 * 24,)
    assert names["l1.mix.right.i"] == (2, 128) and names["l1.mix.right.f.b"] == (2,)
    assert names["l1.mlp.e5.up"] == (32, 128) and names["l1.mlp.e5.down"] == (128, 32) and names["l1.mlp.correction"] == (6,)
    assert "l1.mlp.e0.gate" not in names and "l1.norm2" not in names and names["l2.mix.sink"] == (4,) and "l2.mix.g" not in names
    assert not any(n.startswith("l2.mlp") for n in names) and names["l0.mlp.gate"] == (192, 128) and names["head"] == (320, 128)
    needs = model.cache_needs()
    assert isinstance(needs[1], CompositeNeed) and isinstance(needs[1].members[1], StateNeed)
    left = needs[1].members[0]
    assert (left.window, left.keep_first, left.chunk) == (24, 3, None) and (needs[2].window, needs[2].chunk) == (None, 40)
    assert isinstance(needs[0], PagedNeed) and [t.shape for t in needs[0].tensors] == [(4, 32), (2, 64)]      # two maps' keys, one set of values
    assert needs[0].window is None and needs[0].chunk is None


# ---------------------------------------------------------------------------- the cache manager
def test_a_window_keeps_the_first_pages_and_gives_back_the_middle():
    from llmx_amd.cache import CacheManager, GroupSpec
    g = GroupSpec("win", 4, 64, window=6, keep_first=5)
    m = CacheManager([g], max_requests=1)
    m.open("r")
    m.prepare("r", 30)
    m.commit("r")
    table = m.table("r", 0)
    # the next row (position 30) reads keys 25.. and 0..4: pages 0 and 1 kept, pages 2..5 given back, page 6 (24..27) on
    assert [p >= 0 for p in table] == [True, True, False, False, False, False, True, True]
    assert m.pages_in_use(0) == 4
    assert g.peak_pages(1000, 8) == g.pages_for(14) + 1 + 2 and g.first_read(30) == 25
    m.close("r")
    assert m.pages_in_use(0) == 0


def test_chunks_give_back_the_chunks_before():
    from llmx_amd.cache import CacheManager, GroupSpec
    from llmx_amd.cache.pages import CacheLogicError
    g = GroupSpec("chunks", 4, 64, chunk=10)
    m = CacheManager([g, GroupSpec("all", 4, 64)], max_requests=1)
    m.open("r")
    for n in (9, 1, 13):
        m.prepare("r", n)
        m.commit("r")
    # 23 tokens: the next row sits in the chunk 20..29, so pages below position 20 are given back
    assert [p >= 0 for p in m.table("r", 0)] == [False] * 5 + [True] and all(p >= 0 for p in m.table("r", 1))
    assert g.first_read(19) == 10 and g.first_read(20) == 20 and g.peak_pages(1000, 8) == g.pages_for(18) + 1
    with pytest.raises(CacheLogicError):
        m.truncate("r", 19)               # the row at 19 would read keys from 10 on, which are gone
    m.truncate("r", 21)
    m.close("r")
    assert m.pages_in_use(0) == 0 and m.pages_in_use(1) == 0
