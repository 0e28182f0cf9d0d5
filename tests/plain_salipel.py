"""Salipel computed plainly: whole sequences, float64, no cache, one function a mechanism.

This file shares no code with `llmx_amd`; it reads a configuration (a dict with config.json's keys) and a dict of numpy
arrays by the model folder's tensor names.  Notation: T tokens, E the model's width, H query heads, G key/value heads, D
key width, V value width, F an inner feed-forward width; weights are [out, in] and applied as x @ W.T.

A layer:      h = N(x); x <- x + m (mixer(h) + ff(h))          N(y) = y / rms(y) * w, one norm for both sublayers
Mixers:       "attention":   softmax attention inside chunks of the sequence, a distance penalty a head, unit-RMS values, a
                             sink in the softmax's denominator
              "attention_2": two causal softmax maps a head over one set of values, scores soft-capped, second map
                             subtracted lambda times, the difference normed and gated
              "parallel":    softmax attention over a sliding window that also keeps the sequence's first tokens (values =
                             the projected keys, output gated) beside a matrix memory with exponential gates, summed with
                             two constant weights
Feed-forward: dense gated unit with the tanh form of gelu, or the `top` best experts of relu-squared units (softmax
              scores; a correction on the choice only), or none
Output:       N, then an untied head
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------------------- small pieces
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def log_sigmoid(z):
    return -(np.log1p(np.exp(-np.abs(z))) + np.maximum(-z, 0.0))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def softmax_rows(s, extra=None):
    """Softmax over the last axis of s (masked entries are -inf); `extra` [...] is one more logit a row that only enters
    the denominator."""
    top = s.max(axis=-1, keepdims=True)
    if extra is not None:
        top = np.maximum(top, extra[..., None])
    e = np.exp(s - top)
    den = e.sum(axis=-1, keepdims=True)
    if extra is not None:
        den = den + np.exp(extra[..., None] - top)
    return e / den


# ---------------------------------------------------------------------------- rotation
def wavelength_scaled_frequencies(dims, base, scaling):
    """f_i = base^(-2i/dims) for the dims/2 pairs; with scaling {factor, low, high, original} a pair whose wavelength
    2 pi / f is below original/high keeps f, above original/low it turns `factor` times slower, between them the blend
    weight of the unscaled f is (original/wavelength - low) / (high - low)."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = np.empty_like(f)
    for j, fj in enumerate(f):
        wavelength = 2.0 * math.pi / fj
        if wavelength < original / high:
            out[j] = fj
        elif wavelength > original / low:
            out[j] = fj / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[j] = (1.0 - s) * fj / factor + s * fj
    return out


def rotate_halves(x, positions, rot):
    """x [T, ..., D]: dims (i, i + dims/2), i < dims/2, turn by positions * f_i; dims beyond `dims` pass."""
    dims = int(rot["dims"])
    if dims == 0:
        return x
    f = wavelength_scaled_frequencies(dims, rot["base"], rot.get("scaling"))
    angle = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = np.cos(angle).reshape(shape), np.sin(angle).reshape(shape)
    half = dims // 2
    out = x.copy()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# ---------------------------------------------------------------------------- masks
def mask_causal(T):
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return j <= i


def mask_window_keep_first(T, size, keep_first):
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def mask_chunks(T, size):
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def masked_softmax_attention(q, k, v, scale, mask, transform=None, bias=None, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, V], mask [T, T]; head h reads key/value head h // (H / G).  Scores q.k * scale,
    then `transform` (elementwise), minus `bias` [H, T, T]; softmax over the visible keys, `sink` [H] entering the denominator.
    Returns [T, H, V]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if transform is not None:
            s = transform(s)
        if bias is not None:
            s = s - bias[h]
        s = np.where(mask, s, -np.inf)
        w = softmax_rows(s, None if sink is None else np.full(T, float(sink[h])))
        out[:, h] = w @ v[:, g]
    return out


# ---------------------------------------------------------------------------- mixers
def window_attention(h, W, p, cfg, eps):
    """The windowed attention whose values are its projected keys (before their norm and rotation)."""
    T = h.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (h @ W[p + "q"].T).reshape(T, H, D)
    k = (h @ W[p + "k"].T).reshape(T, G, D)
    v = k.reshape(T, G, V)
    positions = np.arange(T)
    qn = rotate_halves(rms_norm(q, W[p + "q.norm"], eps), positions, cfg["rot"])
    kn = rotate_halves(rms_norm(k, W[p + "k.norm"], eps), positions, cfg["rot"])
    mask = mask_window_keep_first(T, cfg["mask"]["size"], cfg["mask"].get("keep_first", 0))
    o = masked_softmax_attention(qn, kn, v, cfg["scale"], mask).reshape(T, H * V)
    return (o * sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def matrix_memory(h, W, p, cfg, eps, state=None):
    """The matrix memory with exponential input gate and sigmoid forget gate, kept stable by a running maximum that
    starts at zero.  state: (S [H, D, V], n [H, D], m [H]) to continue from; returns (result, state)."""
    T = h.shape[0]
    H, D, V, cap = cfg["heads"], cfg["dim"], cfg["vdim"], float(cfg["gate_cap"])
    q = (h @ W[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, D)
    v = (h @ W[p + "v"].T).reshape(T, H, V)
    gi = cap * np.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    gf = log_sigmoid(cap * np.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    if state is None:
        S, n, m = np.zeros((H, D, V)), np.zeros((H, D)), np.zeros(H)
    else:
        S, n, m = (np.array(s, dtype=np.float64) for s in state)
    o = np.zeros((T, H, V))
    for t in range(T):
        for a in range(H):
            m_new = max(gf[t, a] + m[a], gi[t, a])
            keep, take = math.exp(gf[t, a] + m[a] - m_new), math.exp(gi[t, a] - m_new)
            S[a] = keep * S[a] + take * np.outer(k[t, a], v[t, a])
            n[a] = keep * n[a] + take * k[t, a]
            m[a] = m_new
            o[t, a] = (S[a].T @ q[t, a]) / (max(abs(n[a] @ q[t, a]), math.exp(-m_new)) + 1e-6)
    y = rms_unit(o, eps).reshape(T, H * V) * W[p + "norm"] * sigmoid(h @ W[p + "g"].T)
    return y @ W[p + "o"].T, (S, n, m)


def side_by_side(h, W, p, cfg, eps):
    left = window_attention(h, W, p + "left.", cfg["left"], eps)
    right, _ = matrix_memory(h, W, p + "right.", cfg["right"], eps)
    return cfg["left_scale"] * left + cfg["right_scale"] * right


def distance_slopes(H):
    return np.array([2.0 ** (-8.0 * (a + 1) / H) for a in range(H)])


def chunk_attention(h, W, p, cfg, eps):
    """Attention inside chunks counted from the sequence's start: no rotation, a penalty slope_h (i - j), values of unit
    RMS, a sink a head in the denominator."""
    T = h.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (h @ W[p + "q"].T).reshape(T, H, D)
    k = (h @ W[p + "k"].T).reshape(T, G, D)
    v = rms_unit((h @ W[p + "v"].T).reshape(T, G, V), eps)
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    bias = distance_slopes(H)[:, None, None] * (i - j)[None]
    o = masked_softmax_attention(q, k, v, cfg["scale"], mask_chunks(T, cfg["mask"]["size"]), bias=bias, sink=W[p + "sink"])
    return o.reshape(T, H * V) @ W[p + "o"].T


def difference_lambda(W, p, diff):
    return math.exp(float(W[p + "lq1"] @ W[p + "lk1"])) - math.exp(float(W[p + "lq2"] @ W[p + "lk2"])) + diff


def difference_attention(h, W, p, cfg, eps):
    """Two causal maps a head ([map 1 | map 2] in q's and k's rows) over the same values: a1 - lambda a2, divided by its
    root mean square, times (1 - diff), gated."""
    T = h.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    diff, cap = float(cfg["diff"]), cfg.get("softcap")
    q = (h @ W[p + "q"].T).reshape(T, H, 2, D)
    k = (h @ W[p + "k"].T).reshape(T, G, 2, D)
    v = (h @ W[p + "v"].T).reshape(T, G, V)
    positions = np.arange(T)
    q = rotate_halves(rms_norm(q, W[p + "q.norm"], eps), positions, cfg["rot"])
    k = rotate_halves(rms_norm(k, W[p + "k.norm"], eps), positions, cfg["rot"])
    maps = [masked_softmax_attention(q[:, :, a], k[:, :, a], v, cfg["scale"], mask_causal(T), transform=None if cap is None else (lambda s: cap * np.tanh(s / cap)))
            for a in range(2)]
    o = maps[0] - difference_lambda(W, p, diff) * maps[1]
    o = rms_unit(o, eps) * (1.0 - diff)
    return (o.reshape(T, H * V) * sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


# ---------------------------------------------------------------------------- feed-forward
def dense_unit(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, cfg):
    """(ids [T, top], weights [T, top], logits [T, X]): softmax scores; the `top` largest of score + correction (the lowest
    id first among equals); weights the picked scores over their sum, times the router's scale."""
    r = cfg["router"]
    z = h @ W[p + "router"].T
    s = softmax_rows(z)
    choice = s + W[p + "correction"]
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, : r["top"]]
    picked = np.take_along_axis(s, ids, axis=-1)
    return ids, picked / (picked.sum(axis=-1, keepdims=True) + 1e-20) * r["scale"], z


def routed_units(h, W, p, cfg, picks=None):
    ids, weights, _ = route(h, W, p, cfg)
    if picks is not None:          # the picks are handed in; the weights are still this file's scores of those experts
        ids = np.asarray(picks)
        s = softmax_rows(h @ W[p + "router"].T)
        picked = np.take_along_axis(s, ids, axis=-1)
        weights = picked / (picked.sum(axis=-1, keepdims=True) + 1e-20) * cfg["router"]["scale"]
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for slot, e in enumerate(ids[t]):
            a = np.maximum(W[f"{p}e{e}.up"] @ h[t], 0.0) ** 2
            out[t] += weights[t, slot] * (W[f"{p}e{e}.down"] @ a)
    return out


# ---------------------------------------------------------------------------- the model
MIXERS = {"attention": chunk_attention, "attention_2": difference_attention, "parallel": side_by_side}


def layer(x, W, i, config, picks=None):
    entry, eps = config["layers"][i], config["norm"]["eps"]
    h = rms_norm(x, W[f"l{i}.norm1"], eps)
    y = MIXERS[entry["type"]](h, W, f"l{i}.mix.", entry["mixer"], eps)
    mlp = entry.get("mlp")
    if mlp is not None:
        if mlp["kind"] == "dense":
            y = y + dense_unit(h, W, f"l{i}.mlp.")
        else:
            y = y + routed_units(h, W, f"l{i}.mlp.", mlp, picks)
    return x + config["residual_mult"] * y


def forward(config, W, tokens, picks=None, layers_out=None):
    """Logits [T, vocab] of the whole sequence; `picks` {layer: ids [T, top]} replaces the router's choice in those layers;
    `layers_out` (a list) receives the residual after every layer."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    x = W["embed"][np.asarray(tokens)]
    for i in range(len(config["layers"])):
        x = layer(x, W, i, config, None if picks is None else picks.get(i))
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, W["final.norm"], config["norm"]["eps"]) @ W["head"].T
