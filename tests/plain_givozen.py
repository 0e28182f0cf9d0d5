"""Givozen computed plainly: whole sequences, float64, no cache, one function a mechanism.

This file shares no code with `llmx_amd`; it reads a configuration (a dict with config.json's keys) and a dict of numpy
arrays by the model folder's tensor names.  Notation: T tokens, E the model's width, H query heads, G key/value heads, D
key width, V value width, F an inner feed-forward width; weights are [out, in] and applied as x @ W.T.

A layer:      x <- x + N1b(mixer(N1(x))) ; x <- x + N2b(ff(N2(x)))        N(y) = y / rms(y) * (1 + w)
Mixer:        causal grouped-query softmax attention: biased q, k, v; a partial rotation in halves whose frequencies are
              rescaled by wavelength; a temperature a head on the scores; a sigmoid gate a head on the output
Feed-forward: dense with a polynomial of three unit-RMS powers between its two products, or the `top` best-scored
              experts (sigmoid scores, the score multiplying the expert's *input*) plus a gated shared expert; or none
Loop:         layers start..stop-1 run `times` times; before pass t > 0 the embedding rows are added again, and before
              every pass the pass's own vector
Output:       N, then the embedding table as the head
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------------------- small pieces
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight lies around zero: unit-RMS x times (1 + w)."""
    return rms_unit(x, eps) * (1.0 + w)


# ---------------------------------------------------------------------------- rotation
def wavelength_scaled_frequencies(dims, base, scaling):
    """Frequency of each of the dims/2 pairs: f_i = base^(-2i/dims); with scaling {factor, low, high, original} a pair
    whose wavelength 2 pi / f is shorter than original/high keeps f, one longer than original/low turns `factor` times
    slower, and between the two the blend weight is s = (original/wavelength - low) / (high - low)."""
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


def rotate_halves(x, positions, dims, base, scaling):
    """x [T, heads, D]: dims (i, i + dims/2), i < dims/2, of every head turn by positions * f_i; dims beyond `dims` pass."""
    if dims == 0:
        return x
    f = wavelength_scaled_frequencies(dims, base, scaling)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]          # [T, dims/2]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    half = dims // 2
    out = x.copy()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# ---------------------------------------------------------------------------- attention
def causal_attention(q, k, v, scale, temperature):
    """q [T, H, D], k [T, G, D], v [T, G, V], temperature [H]: row i attends to rows j <= i; head h reads key/value head
    h // (H / G); scores are q.k * scale * temperature[h].  Returns [T, H, V]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    mask = np.tril(np.ones((T, T), dtype=bool))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale * temperature[h]
        s = np.where(mask, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def attention_mixer(h, w, prefix, m, positions):
    """h [T, E] -> [T, E].  m: the layer's `mixer` entry."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T + w[prefix + "q.b"]).reshape(T, H, D)
    k = (h @ w[prefix + "k"].T + w[prefix + "k.b"]).reshape(T, G, D)
    v = (h @ w[prefix + "v"].T + w[prefix + "v.b"]).reshape(T, G, V)
    rot = m["rot"]
    q = rotate_halves(q, positions, rot["dims"], rot["base"], rot.get("scaling"))
    k = rotate_halves(k, positions, rot["dims"], rot["base"], rot.get("scaling"))
    o = causal_attention(q, k, v, m["scale"], w[prefix + "temp"])
    o = o * sigmoid(h @ w[prefix + "g"].T)[:, :, None]
    return o.reshape(T, H * V) @ w[prefix + "o"].T


# ---------------------------------------------------------------------------- feed-forward
def poly_norm(z, abce, eps):
    """a U(z) + b U(z^2) + c U(z^3) + e, powers taken element by element, U dividing a row by its root mean square."""
    a, b, c, e = (float(t) for t in abce)
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e


def dense_ff(h, w, prefix, eps):
    return poly_norm(h @ w[prefix + "up"].T, w[prefix + "act"], eps) @ w[prefix + "down"].T


def clamped_glu_expert(h, w, prefix, limit):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = np.minimum(h @ w[prefix + "gate"].T, limit)
    u = np.clip(h @ w[prefix + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[prefix + "down"].T


def route(h, w_router, top):
    """Scores sigmoid(W_router h); the `top` largest of a row (the lower id on equal scores) and their scores."""
    s = sigmoid(h @ w_router.T)
    order = np.argsort(-s, axis=1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, axis=1), s


def moe_ff(h, w, prefix, mlp, picks=None):
    """Sum over a row's picked experts of expert(score * h), plus sigmoid(W_sg h) * shared(h) where there is a shared
    expert.  `picks` [T, top] replaces the router's choice (the scores stay the router's own)."""
    T = h.shape[0]
    top = mlp["router"]["top"]
    ids, scores, s_all = route(h, w[prefix + "router"], top)
    if picks is not None:
        ids = np.asarray(picks)
        scores = np.take_along_axis(s_all, ids, axis=1)
    out = np.zeros((T, w[prefix + "e0.down"].shape[0]))
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += clamped_glu_expert(scores[t, j] * h[t:t + 1], w, f"{prefix}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        gate = sigmoid(h @ w[prefix + "shared.sg"].T)                      # [T, 1]
        out += gate * clamped_glu_expert(h, w, prefix + "shared.", mlp["shared"]["limit"])
    return out


# ---------------------------------------------------------------------------- the model
def run_order(config):
    """[(layer, pass number or None, first of its pass)] in the order the layers run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None, False) for i in range(start)]
    for t in range(times):
        order += [(i, t, i == start) for i in range(start, stop)]
    return order + [(i, None, False) for i in range(stop, n)]


def forward(config, w, tokens, picks=None, keep_layers=False):
    """Logits [T, vocab] of one sequence; with keep_layers also the residual after every layer run.  `picks`:
    {index in the run order: [T, top]} replaces the router's choice in those routed layer runs."""
    eps = config["norm"]["eps"]
    positions = np.arange(len(tokens))
    emb = w["embed"][np.asarray(tokens)]
    x = emb.copy()
    layers = []
    for at, (i, t, first) in enumerate(run_order(config)):
        if first:
            if t > 0:
                x = x + emb
            x = x + w["loop.step"][t]
        layer = config["layers"][i]
        p = f"l{i}."
        y = attention_mixer(offset_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], positions)
        x = x + offset_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            h = offset_norm(x, w[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = dense_ff(h, w, p + "mlp.", eps)
            else:
                y = moe_ff(h, w, p + "mlp.", mlp, None if picks is None else picks.get(at))
            x = x + offset_norm(y, w[p + "norm2b"], eps)
        layers.append(x.copy())
    logits = offset_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, np.stack(layers)) if keep_layers else logits
