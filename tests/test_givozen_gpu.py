"""Givozen in the engine against the plain implementation (tests/plain_givozen.py), mechanism by mechanism and whole.

Kernels alone (the polynomial of unit-RMS powers, the gated unit with a factor on its input and a switch on its result, the
gate a head, the pass vector, the norm with an offset weight and its join, the combine with unit weights, the attention step
with biases, a temperature a head and further columns behind v) against the plain functions; one query made to fit a single
key far back, at page borders and among the first tokens, in a prompt's rows and decoded alone; then the engine under every
way of cutting the same tokens into steps, which must agree bit for bit with each other in both dtypes, with the plain
implementation within F32_TOL in float32 and within BF16_TOL in bfloat16 (the engine's expert picks handed over); pages
and request seats that are used again; long decoding; greedy generation through `generate`; the trace replay tool and the
command line.
"""

from __future__ import annotations

import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_givozen as plain
from givozen_cases import CONFIGS, PAGES, greedy, load_plain, model_folder, plain_logits, portions, routed_runs, tokens_for, write_folder

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # |engine - plain| over all logits relative to the largest |logit|: float32 sums in another order
BF16_TOL = 5e-2     # the serving path against the plain implementation (float64, nothing rounded), with the engine's expert picks
BF16_RMS = 2.5e-2   # ... and the root mean square of all differences relative to that of the logits
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def ops():
    from llmx_amd import ops as o
    return o


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(device="cuda", dtype=dtype).contiguous()


def close(got, want, tol, what=""):
    got, want = torch.as_tensor(np.asarray(got.cpu() if isinstance(got, torch.Tensor) else got)).double(), torch.as_tensor(np.asarray(want.cpu() if isinstance(want, torch.Tensor) else want)).double()
    err = float((got - want).abs().max()) / max(float(want.abs().max()), 1e-30)
    assert err <= tol, f"{what}: relative error {err:.3e} above {tol:.1e}"
    return err


# ---------------------------------------------------------------------------
# kernels alone
@pytest.mark.parametrize("rows,n", [(1, 8), (5, 21), (3, 1030), (2, 4100), (2, 16384), (2, 16391)])
def test_polynomial_of_unit_rms_powers(rows, n):
    rng = np.random.default_rng(n)
    o = ops()
    z = rng.normal(size=(rows, n)) * 1.7
    abce = np.array([0.6, -0.9, 0.3, 0.2])
    for eps in (1e-6, 0.5):
        out = torch.empty(rows, n, device="cuda")
        o.act_polynorm(dev(z), dev(abce), eps, out)
        close(out, plain.poly_norm(z.astype(np.float32).astype(np.float64), abce.astype(np.float32), eps), 3e-6, f"eps {eps}")
    out16 = torch.empty(rows, n, device="cuda", dtype=torch.bfloat16)
    o.act_polynorm(dev(z), dev(abce), 1e-6, out16)
    close(out16.float(), plain.poly_norm(z, abce, 1e-6), 8e-3)


@pytest.mark.parametrize("kind", ["clamped", "silu"])
def test_gated_unit_with_a_factor_on_its_input_and_a_switch(kind):
    rng = np.random.default_rng(7)
    o = ops()
    P, n, limit = 13, 37, 0.8
    pre = rng.normal(size=(P, 2 * n + 3)) * 2                    # further columns behind the up values are left alone
    scale = rng.uniform(0.1, 1.0, size=P)
    wide = rng.normal(size=(P, 5))
    gate_logit = wide[:, 3:4]
    g, u = pre[:, :n] * scale[:, None], pre[:, n:2 * n] * scale[:, None]
    if kind == "clamped":
        gc, uc = np.minimum(g, limit), np.clip(u, -limit, limit)
        want = gc * plain.sigmoid(1.702 * gc) * (uc + 1.0)
    else:
        want = g * plain.sigmoid(g) * u
    want_switched = want * plain.sigmoid(gate_logit)
    code = o.GLU_CLAMPED if kind == "clamped" else o.GLU_SILU
    out = torch.empty(P, n, device="cuda")
    o.act_glu(dev(pre), o.Glu(code, limit, dev(scale)), out)
    close(out, want, 3e-6)
    wide_d = dev(wide)
    o.act_glu(dev(pre), o.Glu(code, limit, dev(scale), wide_d[:, 3:4]), out)
    close(out, want_switched, 3e-6)
    o.act_glu(dev(pre), o.Glu(code, limit), out)                  # no factor: 1
    plain_g, plain_u = pre[:, :n], pre[:, n:2 * n]
    if kind == "clamped":
        gc, uc = np.minimum(plain_g, limit), np.clip(plain_u, -limit, limit)
        close(out, gc * plain.sigmoid(1.702 * gc) * (uc + 1.0), 3e-6)
    else:
        close(out, plain_g * plain.sigmoid(plain_g) * plain_u, 3e-6)


@pytest.fixture(params=[True, False], ids=["in the epilogue", "a kernel of its own"])
def unit_in_epilogue(request):
    o = ops()
    before = o.GLU_IN_EPILOGUE
    o.GLU_IN_EPILOGUE = request.param
    yield request.param
    o.GLU_IN_EPILOGUE = before


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_products_with_a_gated_unit_dense_and_grouped(dtype, unit_in_epilogue):
    """gemm and grouped_gemm with a gated unit (clamped, a factor on each row's input, a switch on its result) against the
    plain expert, at a few row counts (the weight-streaming and the tiled products) and widths; the unit in the products'
    epilogue, and as a kernel of its own behind a storing product."""
    rng = np.random.default_rng(11)
    o = ops()
    o.take_launches()
    tol = 2e-5 if dtype == torch.float32 else 2.5e-2
    for rows, E, F in ((1, 64, 32), (9, 128, 48), (70, 64, 96), (300, 128, 256)):
        h = rng.normal(size=(rows, E))
        wg, wu = rng.normal(size=(F, E)) * 0.2, rng.normal(size=(F, E)) * 0.2
        w = {"e.gate": wg, "e.up": wu, "e.down": np.eye(F)}
        switch = rng.normal(size=(rows, 1))
        out = torch.empty(rows, F, device="cuda", dtype=dtype)
        o.gemm(dev(h, dtype), dev(np.concatenate([wg, wu]), dtype), out, o.EPI_SWIGLU, glu=o.Glu(o.GLU_CLAMPED, 0.9, None, dev(switch)))
        hr = dev(h, dtype).double().cpu().numpy()
        wr = {k: dev(v, dtype).double().cpu().numpy() for k, v in w.items()}
        close(out.float(), plain.sigmoid(switch) * plain.clamped_glu_expert(hr, wr, "e.", 0.9), tol, f"dense {rows}x{E}x{F}")
        # grouped: X experts, two picks a row, the score a factor on the pair's input
        X, k = 5, 2
        wgu = rng.normal(size=(X, 2 * F, E)) * 0.2
        ids = np.stack([rng.permutation(X)[:k] for _ in range(rows)]).astype(np.int32)
        score = rng.uniform(0.2, 1.0, size=(rows, k))
        idd = dev(ids, torch.int32)
        counts, offsets = torch.empty(X, dtype=torch.int32, device="cuda"), torch.empty(X + 1, dtype=torch.int32, device="cuda")
        pairs, active = torch.empty(rows * k, dtype=torch.int32, device="cuda"), torch.empty(X, dtype=torch.int32, device="cuda")
        n_active = torch.empty(1, dtype=torch.int32, device="cuda")
        o.moe_align(idd, X, counts, offsets, pairs, active, n_active)
        act = torch.empty(rows * k, F, device="cuda", dtype=dtype)
        o.grouped_gemm(dev(h, dtype), dev(wgu, dtype), act, offsets, pairs, k, o.EPI_SWIGLU, active, n_active, token_rows=rows,
                       glu=o.Glu(o.GLU_CLAMPED, 1.3, dev(score).view(rows * k)))
        wgur = dev(wgu, dtype).double().cpu().numpy()
        for t in range(rows):
            for j in range(k):
                e = int(ids[t, j])
                we = {"x.gate": wgur[e, :F], "x.up": wgur[e, F:], "x.down": np.eye(F)}
                want = plain.clamped_glu_expert(np.float32(score[t, j]) * hr[t:t + 1], we, "x.", 1.3)[0]
                close(act[t * k + j].float(), want, tol, f"grouped row {t} slot {j}")
    assert bool(o.take_launches().get("act.glu")) == (not unit_in_epilogue)


def test_gate_a_head_pass_vector_offset_norm_and_unit_combine():
    rng = np.random.default_rng(3)
    o = ops()
    T, H, V, E = 6, 3, 5, 22
    vals, proj = rng.normal(size=(T, H * V)), rng.normal(size=(T, 40))
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        got = dev(vals, dtype)
        o.gate_heads(got, dev(proj)[:, 31:31 + H], H)
        want = dev(vals, dtype).double().cpu().numpy().reshape(T, H, V) * plain.sigmoid(proj[:, 31:31 + H])[:, :, None]
        close(got.float(), want.reshape(T, H * V), tol, "gate a head")
    x, rows, vec = rng.normal(size=(T, E)), rng.normal(size=(T, E)), rng.normal(size=(2, E))
    xd, vd = dev(x), dev(vec)
    o.add_rows_vector(xd, dev(rows), vd[1])
    close(xd, x + rows + vec[1], 1e-6)
    o.add_rows_vector(xd, None, vd[0])
    close(xd, x + rows + vec[1] + vec[0], 1e-6)
    # the norm part with a weight stored around zero, and its join into the residual
    from llmx_amd.parts.base import BuildContext, build_part
    from llmx_amd.parts.spec import PartSpec
    part = build_part("norm", PartSpec("rmsnorm", {"width": E, "eps": 1e-3, "tensor": "", "offset": 1.0}, "n"),
                      BuildContext(torch.float32, torch.device("cuda"), 8, 16))
    w = rng.normal(size=E) * 0.2
    part.load({"n": dev(w)})
    out = torch.empty(T, E, device="cuda")
    part.forward(None, dev(x), out)
    close(out, plain.offset_norm(x, w.astype(np.float32), 1e-3), 2e-6)
    res = dev(rows)
    part.add_into(None, res, dev(x))
    close(res, rows + plain.offset_norm(x, w.astype(np.float32), 1e-3), 2e-6)
    # the combine with every weight 1
    k = 3
    y, ids = rng.normal(size=(T * k, E)), np.tile(np.arange(k, dtype=np.int32), (T, 1))
    acc = dev(x)
    o.moe_combine(acc, dev(y), dev(ids, torch.int32), None, accumulate=True)
    close(acc, x + y.reshape(T, k, E).sum(1), 2e-6)


@pytest.mark.parametrize("rows,n", [(1, 8), (5, 54), (3, 1030), (2, 8200)])
def test_join_and_next_norm_in_one_launch(rows, n):
    """x += N_join(y); h = N_next(x) as one kernel: the plain functions' values, and bit for bit the join kernel followed by
    the norm kernel (a block may use either way for the same place in the model)."""
    rng = np.random.default_rng(n + rows)
    o = ops()
    x, y = rng.normal(size=(rows, n)) * 3, rng.normal(size=(rows, n)) * 0.5
    wj, wn = 1.0 + rng.normal(size=n) * 0.2, 1.0 + rng.normal(size=n) * 0.2
    xd, h16, h32 = dev(x), torch.empty(rows, n, device="cuda", dtype=torch.bfloat16), torch.empty(rows, n, device="cuda")
    o.rmsnorm_add_norm(xd, dev(y), dev(wj), 1e-5, dev(wn), 1e-3, h16, h32)
    f32 = lambda a: np.asarray(a, dtype=np.float32).astype(np.float64)
    want_x = f32(x) + plain.rms_unit(f32(y), 1e-5) * f32(wj)
    close(xd, want_x, 2e-6, "the joined rows")
    close(h32, plain.rms_unit(want_x, 1e-3) * f32(wn), 3e-6, "their norm")
    assert torch.equal(h16, h32.to(torch.bfloat16))
    x2, g32 = dev(x), torch.empty(rows, n, device="cuda")
    o.rmsnorm_add(x2, dev(y), dev(wj), 1e-5)
    o.rmsnorm(x2, dev(wn), 1e-3, None, g32)
    assert torch.equal(x2, xd) and torch.equal(g32, h32)


def _attention_case(dtype, H, G, D, VD, R, scaling, page, length, sharp=None, decode_from=None, scale=0.3):
    """One attention part alone through its kernels (the step with biases and a temperature a head, the attention over
    shuffled pages, the gate a head) against the plain mixer.  sharp = (row, key): the row's query is made to fit that key
    alone.  decode_from: rows from there on are run one by one, each in a launch of its own, as decoded tokens are."""
    from llmx_amd.parts.position import scaled_table
    rng = np.random.default_rng(H * 1000 + D + length)
    o = ops()
    E = 24
    sc = dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": VD, "scale": scale, "rot": {"base": 500.0, "dims": R, "scaling": sc}}
    w = {"p." + n: rng.normal(size=s) * 0.5 for n, s in (("q", (H * D, E)), ("k", (G * D, E)), ("v", (G * VD, E)), ("q.b", (H * D,)), ("k.b", (G * D,)),
                                                         ("v.b", (G * VD,)), ("g", (H, E)))}
    w["p.temp"] = rng.uniform(0.5, 1.6, size=H)
    w["p.o"] = np.eye(H * VD)
    h = rng.normal(size=(length, E))
    if sharp is not None:
        # the key row's input is far from all others and the query row's input is the same; every query head is made the
        # key head's projection, so that key's score stands out as far as the rotation lets it
        row, key = sharp
        h[key] = h[key] * 5
        h[row] = h[key]
        w["p.q"] = np.concatenate([w["p.k"][(hh // (H // G)) * D:(hh // (H // G) + 1) * D] for hh in range(H)]) * 4.0
        w["p.q.b"] = np.concatenate([w["p.k.b"][(hh // (H // G)) * D:(hh // (H // G) + 1) * D] for hh in range(H)]) * 4.0
    want = plain.attention_mixer(h, w, "p.", m, np.arange(length))
    width = H * D + G * D + G * VD
    proj = np.concatenate([h @ w["p.q"].T, h @ w["p.k"].T, h @ w["p.v"].T, h @ w["p.g"].T], axis=1)
    bias = np.concatenate([w["p.q.b"], w["p.k.b"], w["p.v.b"]])
    n_pages = -(-length // page)
    order = list(range(n_pages + 3))
    random.Random(length).shuffle(order)
    tables = dev(np.array([order[:n_pages] + [-1] * 5]), torch.int32)
    kc = torch.zeros(n_pages + 3, G, page, D, device="cuda", dtype=dtype)
    vc = torch.zeros(n_pages + 3, G, VD, page, device="cuda", dtype=dtype)
    cos_sin = dev(scaled_table(length, R, 500.0, sc))
    temp = dev(w["p.temp"])
    out = torch.empty(length, H * VD, device="cuda", dtype=dtype)
    runs = [(0, length)] if decode_from is None else [(0, decode_from)] + [(i, i + 1) for i in range(decode_from, length)]
    for a, b in runs:
        n = b - a
        pos, ent = dev(np.arange(a, b), torch.int32), dev(np.zeros(n), torch.int32)
        rows = dev(proj[a:b])
        q = torch.empty(n, H * D, device="cuda", dtype=dtype)
        o.head_norm_rope_kvwrite(rows, dev(bias), None, None, cos_sin, pos, ent, tables, q, kc, vc, 0.0, H, G, D, R, o.QKNORM_NONE,
                                 pairing=o.ROPE_HALVES, q_scale=temp)
        part = torch.empty(n, H * VD, device="cuda", dtype=dtype)
        plan = None
        if VD == D and o.attention_mfma_ok(dtype, D, page):
            plan = o.attention_plan([n], [b], H, G, torch.device("cuda"), 0)
        o.paged_attention(q, kc, vc, pos, ent, tables, part, scale, H, plan=plan, head_gate=rows[:, width:])
        out[a:b] = part
    return out.float().cpu(), torch.as_tensor(want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 32, 16, (4.0, 1.0, 4.0, 64), 16), (3, 1, 10, 6, 6, None, 4), (6, 6, 16, 48, 16, (8.0, 2.0, 16.0, 32), 16),
                                   (8, 4, 64, 64, 32, (4.0, 1.0, 8.0, 128), 16), (1, 1, 128, 128, 0, None, 16), (2, 1, 48, 16, 48, None, 8)])
def test_attention_with_biases_temperature_and_gate_over_shuffled_pages(dtype, sizes):
    H, G, D, VD, R, scaling, page = sizes
    scale = 0.5 / D ** 0.5          # scores of the same moderate spread whatever the head's width (the sharp cases are below)
    got, want = _attention_case(dtype, H, G, D, VD, R, scaling, page, 150, scale=scale)
    close(got, want, 2e-5 if dtype == torch.float32 else 2.5e-2, "a prompt's rows")
    got, want = _attention_case(dtype, H, G, D, VD, R, scaling, page, 150, decode_from=120, scale=scale)
    close(got, want, 2e-5 if dtype == torch.float32 else 2.5e-2, "a decoded tail")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("key", [0, 1, 2, 15, 16, 17, 127, 128, 129, 255, 256, 500, 683, 684])
def test_attention_finds_one_key_far_back(dtype, key):
    """A row whose query fits one key among 700: the first tokens, both sides of page borders (16) and of the attention
    kernels' segment borders (128), far back and the row before.  The row's result is then that key's value (times the
    row's gate), in a prompt's rows and when the last rows are decoded alone; values as wide as keys (the matrix cores run
    in bfloat16) and of their own width."""
    for VD, page in ((32, 16), (24, 16)):
        row = 685
        got, want = _attention_case(dtype, 4, 2, 32, VD, 0, None, page, 700, sharp=(row, key))
        close(got[row], want[row], 3e-5 if dtype == torch.float32 else 2.5e-2, f"key {key}, values of {VD}, in a prompt")
        got, want = _attention_case(dtype, 4, 2, 32, VD, 0, None, page, 700, sharp=(row, key), decode_from=680)
        close(got[row], want[row], 3e-5 if dtype == torch.float32 else 2.5e-2, f"key {key}, values of {VD}, decoded")


# ---------------------------------------------------------------------------
# the engine
def make_engine(name, dtype, kv_tokens=1024, max_requests=4, graphs=True, folder=None):
    from llmx_amd.engine import Engine
    return Engine.load(folder or model_folder(name), dtype=dtype, kv_tokens=kv_tokens, page_tokens=PAGES[name], max_requests=max_requests, graphs=graphs)


@pytest.fixture(scope="module", params=[(n, d) for n in CONFIGS for d in ("float32", "bfloat16")], ids=lambda p: f"{p[0]}-{p[1]}")
def setup(request):
    name, dtype = request.param
    return name, dtype, make_engine(name, dtype)


def run_cut(engine, rid, tokens, cuts):
    from llmx_amd.engine import StepEntry
    engine.add_request(rid)
    rows = [engine.step([StepEntry(rid, tokens[a:b], list(range(b - a)))]).clone() for a, b in cuts]
    engine.end_request(rid)
    return torch.cat(rows).cpu()


def same_rows(got, whole, what):
    """Two cuttings of the same tokens give every row the same bits, in both number formats."""
    assert torch.equal(got, whole), f"{what}: rows differ, first at row {int((got != whole).any(1).nonzero()[0])}"


def run_whole_with_picks(engine, tokens):
    """(rows, picks): a whole prompt's logits and, for every routed layer run in order, the experts the engine picked
    [T, top], each row's picks checked against the engine's own float32 router logits (the `top` largest, lower ids first)."""
    shown = []
    engine.observer = lambda step, kind, **t: shown.append((t["ids"].cpu().numpy().copy(), t["logits"].cpu().numpy().copy())) if kind == "routing" else None
    try:
        rows = run_cut(engine, "picks", tokens, [(0, len(tokens))])
    finally:
        engine.observer = None
    for ids, z in shown:
        for t in range(ids.shape[0]):
            assert list(ids[t]) == sorted(range(z.shape[1]), key=lambda e: (-z[t, e], e))[:ids.shape[1]]
    return rows, [ids for ids, _ in shown]


def reference_rows(name, dtype, length, seed, got, engine=None, folder=None, tol=None):
    """float32 against the plain implementation.  bfloat16 too, within BF16_TOL, with the engine's own expert picks handed
    to the plain implementation (a near tie of two router logits may fall the other way after rounding, and then another
    expert runs); `got` must be the bits of the whole prompt that was run to see the picks."""
    tokens = tokens_for(name, length, seed)
    if dtype == "float32":
        want = plain_logits(name, length, seed) if folder is None else plain.forward(*load_plain(folder), tokens)
        close(got, want, tol or F32_TOL, "against the plain implementation")
        return
    rows, picks = run_whole_with_picks(engine, tokens)
    assert torch.equal(rows, got), "the whole prompt run again gives other bits"
    config, tensors = load_plain(folder or model_folder(name))
    want = torch.as_tensor(plain.forward(config, tensors, tokens, picks=dict(zip(routed_runs(config), picks))))
    close(got, want, tol or BF16_TOL, "against the plain implementation with the engine's picks")
    rms = float((got.double() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt())
    assert rms <= BF16_RMS, f"root mean square of the differences {rms:.3e} of the logits' above {BF16_RMS:.1e}"


LENGTHS = (1, 2, 9, 33, 75, 130)


def test_whole_prompts_and_every_layer(setup):
    name, dtype, engine = setup
    for seed, length in enumerate(LENGTHS):
        reference_rows(name, dtype, length, seed, run_cut(engine, ("w", seed), tokens_for(name, length, seed), [(0, length)]), engine)
    if dtype != "float32":
        return
    config, tensors = load_plain(model_folder(name))
    tokens = tokens_for(name, 21, 99)
    _, layers = plain.forward(config, tensors, tokens, keep_layers=True)
    seen = []
    engine.observer = lambda step, kind, **t: seen.append(t["residual"].clone()) if kind == "layer" else None
    try:
        run_cut(engine, "layers", tokens, [(0, 21)])
    finally:
        engine.observer = None
    assert len(seen) == len(layers) == len(plain.run_order(config))
    for i, (got, want) in enumerate(zip(seen, layers)):
        close(got, want, F32_TOL, f"residual after layer run {i}")


def test_prompt_against_token_by_token_and_portions(setup):
    """Every cutting gives every row the same bits: whole, token by token from the first token, most of it whole and the
    rest one by one, portions of changing size down to two tokens and to one, pairs."""
    name, dtype, engine = setup
    length, seed = 130, 5
    tokens = tokens_for(name, length, seed)
    whole = run_cut(engine, "whole", tokens, [(0, length)])
    reference_rows(name, dtype, length, seed, whole, engine)
    cuttings = {
        "one by one": [(i, i + 1) for i in range(length)],
        "decoded tail": [(0, length - 50)] + [(i, i + 1) for i in range(length - 50, length)],
        "portions": portions(length, 1),
        "portions of one": portions(length, 2, smallest=1),
        "pairs": [(i, min(i + 2, length)) for i in range(0, length, 2)],
    }
    for what, cuts in cuttings.items():
        same_rows(run_cut(engine, what, tokens, cuts), whole, what)


def test_unequal_requests_in_one_batch_and_reused_pages_and_seats(setup):
    """Eight requests of unequal length through four seats, portions of some beside single tokens of others, in an engine
    with so few pages that ended requests' pages and seats are taken again by later ones; every row has the bits it has
    when its request runs alone in a fresh engine."""
    from llmx_amd.engine import StepEntry
    name, dtype, _ = setup
    lengths = [70, 23, 1, 96, 40, 17, 64, 5]
    alone_engine = make_engine(name, dtype)
    alone = {i: run_cut(alone_engine, i, tokens_for(name, n, 20 + i), [(0, n)]) for i, n in enumerate(lengths)}
    engine = make_engine(name, dtype, kv_tokens=4 * 112, max_requests=4)
    rng = random.Random(3)
    waiting = list(range(len(lengths)))
    live, fed, got = [], {}, {i: [] for i in range(len(lengths))}
    while waiting or live:
        while waiting and len(live) < 4:
            i = waiting.pop(0)
            engine.add_request(i)
            live.append(i)
            fed[i] = 0
        entries, taken = [], []
        for i in live:
            if rng.random() < 0.2 and len(live) > 1:
                continue                                     # a request may be left out of a step
            left = lengths[i] - fed[i]
            n = 1 if rng.random() < 0.4 else min(left, rng.choice([2, 3, 8, 16, 31]))
            entries.append(StepEntry(i, tokens_for(name, lengths[i], 20 + i)[fed[i]:fed[i] + n], list(range(n))))
            taken.append((i, n))
        if not entries:
            continue
        out = engine.step(entries).clone().cpu()
        at = 0
        for i, n in taken:
            got[i].append(out[at:at + n])
            at += n
            fed[i] += n
            if fed[i] == lengths[i]:
                engine.end_request(i)
                live.remove(i)
    for i in range(len(lengths)):
        same_rows(torch.cat(got[i]), alone[i], f"request {i} in batches against its whole prompt alone")
    assert all(engine.cache.pages_in_use(g) == 0 for g in range(len(engine.cache.groups)))
    assert engine.cache.slots.in_use == 0


def test_long_decoding_and_graph_replays(setup):
    """A short prompt, then 230 tokens one by one over many pages: the rows of the whole sequence, from an engine that
    replays decode steps as graphs and from one that does not."""
    name, dtype, engine = setup
    length, seed = 250, 8
    tokens = tokens_for(name, length, seed)
    cuts = [(0, 20)] + [(i, i + 1) for i in range(20, length)]
    before = engine.graph_replays
    got = run_cut(engine, "long", tokens, cuts)
    assert engine.graphs and engine.graph_replays - before > 150
    eager = make_engine(name, dtype, graphs=False)
    assert torch.equal(run_cut(eager, "long", tokens, cuts), got)
    whole = run_cut(eager, "whole", tokens, [(0, length)])
    same_rows(got, whole, "decoded against whole")
    reference_rows(name, dtype, length, seed, whole, eager)


def test_which_kernels_a_serving_step_takes():
    """The launch witness: at sizes the matrix cores take (configuration A), a bfloat16 step runs the design's own kernels
    and the matrix-core attention and products, never the universal ones; a float32 engine never launches a bfloat16
    product.  A dispatch that fell back silently fails here, not only in a benchmark."""
    from llmx_amd.engine import StepEntry
    o = ops()
    tokens = tokens_for("A", 70, 2)
    for dtype in ("bfloat16", "float32"):
        engine = make_engine("A", dtype, graphs=False)
        engine.add_request("r")
        seen = {}
        for entry in (StepEntry("r", tokens[:69], [68]), StepEntry("r", tokens[69:], [0])):       # a prompt's portion, then one token
            o.take_launches()
            engine.step([entry])
            for name, count in o.take_launches().items():
                seen[name] = seen.get(name, 0) + count
        for name in ("head_norm_rope_kvwrite", "act.polynorm", "add_rows_vector", "rmsnorm_add", "rmsnorm_add_norm", "rmsnorm",
                     "moe_combine"):
            assert seen.get(name), f"{dtype}: no launch of {name} ({sorted(seen)})"
        # the experts' unit runs in their first product's epilogue, the gate a head where the attention stores its result
        assert "act.glu" not in seen and "gate_heads" not in seen
        assert seen["add_rows_vector"] == 2 * 3                                          # three passes, two steps
        assert seen["rmsnorm_add_norm"] == 2 * 7 and seen["rmsnorm_add"] == 2 * 8        # seven runs have a feed-forward; its join and the last layer's
        if dtype == "bfloat16":
            assert not any(n.startswith(("gemm_generic", "attention.generic")) for n in seen), sorted(seen)
            assert any(n.startswith("attention.") for n in seen) and any(n.startswith("gemm_skinny") or n.startswith("gemm_tile") for n in seen)
        else:
            assert not any(n.startswith(("gemm_skinny", "gemm_tile", "attention.tiles", "attention.split", "attention.direct")) for n in seen), sorted(seen)


def test_a_failed_step_leaves_pages_as_they_were():
    from llmx_amd.cache import OutOfPages
    from llmx_amd.engine import StepEntry
    name = "A"
    tokens = tokens_for(name, 60, 1)
    engine = make_engine(name, "float32", kv_tokens=64, max_requests=2)
    engine.add_request("a")
    engine.add_request("b")
    first = engine.step([StepEntry("a", tokens[:20], [19])]).clone()
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("a", tokens[20:40], [19]), StepEntry("b", tokens[:60], [])])
    rest = engine.step([StepEntry("a", tokens[20:60], list(range(40)))]).clone().cpu()
    whole = run_cut(make_engine(name, "float32"), "w", tokens, [(0, 60)])
    assert torch.equal(first.cpu()[0], whole[19]) and torch.equal(rest, whole[20:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_a_long_prompt(dtype, tmp_path):
    """Query and key weights made larger (and the temperatures raised) let the softmax pick single keys hundreds of tokens
    back, so a key lost at a page's or a segment's edge, or a pass that read another pass's cache, shows.  Whole, portions
    and decoding agree bit for bit, and float32 with the plain model."""
    def edit(tensors):
        for k in tensors:
            if k.endswith("mix.q") or k.endswith("mix.k"):
                tensors[k] = (tensors[k].float() * 2.0).to(tensors[k].dtype)
            if k.endswith("mix.temp"):
                tensors[k] = tensors[k] * 1.5
    folder = write_folder(CONFIGS["A"], 27, str(tmp_path / "sharp"), edit)
    engine = make_engine("A", dtype, folder=folder)
    length = 520
    tokens = tokens_for("A", length, 4)
    whole = run_cut(engine, "w", tokens, [(0, length)])
    config, tensors = load_plain(folder)
    if dtype == "float32":
        want = plain.forward(config, tensors, tokens)
        close(whole, want, 1e-4, "against the plain implementation")
        # far keys carry weight indeed: another first token changes the last row
        other = plain.forward(config, tensors, [(tokens[0] + 1) % 320] + tokens[1:])
        assert float(np.abs(other[-1] - want[-1]).max()) > 1e-3 * float(np.abs(want).max())
    else:
        rows, picks = run_whole_with_picks(engine, tokens)
        assert torch.equal(rows, whole)
        # sharp scores amplify every rounding of q and k: the single worst logit gets more room here, the mean stays bound
        want = torch.as_tensor(plain.forward(config, tensors, tokens, picks=dict(zip(routed_runs(config), picks))))
        close(whole, want, 2e-1, "against the plain implementation with the engine's picks")
        rms = float((whole.double() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt())
        assert rms <= 2 * BF16_RMS, f"root mean square of the differences {rms:.3e} of the logits'"
    same_rows(run_cut(engine, "p", tokens, portions(length, 9)), whole, "portions")
    same_rows(run_cut(engine, "pairs", tokens, [(i, i + 2) for i in range(0, length, 2)]), whole, "pairs")
    same_rows(run_cut(engine, "d", tokens, [(0, length - 90)] + [(i, i + 1) for i in range(length - 90, length)]), whole, "decoded")


def test_greedy_generation_through_the_scheduler():
    """`generate` (scheduler, step function, device sampler) with prompts of unequal length and a small step budget, so
    that prompts are cut into portions beside decoding requests; float32 picks the plain implementation's tokens."""
    from llmx_amd import SamplingParams, generate
    name = "A"
    config, tensors = load_plain(model_folder(name))
    prompts = [tokens_for(name, n, 40 + n) for n in (3, 29, 11, 1, 18)]
    engine = make_engine(name, "float32", kv_tokens=512, max_requests=3)
    got = generate(engine, prompts, SamplingParams(max_tokens=10, temp=0.0), max_seqs=3, max_step_tokens=16)
    for p, g in zip(prompts, got):
        assert g == greedy(config, tensors, p, 10)
    # bfloat16: a near tie of two router logits may fall the other way than in the plain model and another expert runs, so
    # the tokens are compared with those the same engine gives step by step without scheduler and sampler (every cutting
    # gives a row the same bits): whole prompt, then one token at a time, the largest logit each time
    engine16 = make_engine(name, "bfloat16", kv_tokens=512, max_requests=3)
    got16 = generate(engine16, prompts, SamplingParams(max_tokens=10, temp=0.0), max_seqs=3, max_step_tokens=16)
    by_hand = make_engine(name, "bfloat16", kv_tokens=512, max_requests=3, graphs=False)
    for i, (p, g) in enumerate(zip(prompts, got16)):
        by_hand.add_request(i)
        row, want = by_hand.prefill(i, p), []
        for _ in range(10):
            want.append(int(torch.argmax(row)))
            row = by_hand.decode_one(i, want[-1])
        by_hand.end_request(i)
        assert g == want


def test_trace_replay_and_command_line(tmp_path):
    """bin/trace_run as a subprocess on a model folder: a prompt portion beside decoded tokens, requests that end and
    whose seats are taken again; the logits files are the plain model's rows.  `llmx logits` reads the same folder."""
    name = "C"
    a, b, c = tokens_for(name, 40, 1), tokens_for(name, 9, 2), tokens_for(name, 30, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[33:34], "want": [0]}, {"id": "b", "tokens": b, "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "c", "tokens": c[:2], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "c", "tokens": c[2:], "want": [27]}, {"id": "a", "tokens": a[34:], "want": [5]}], "end": ["a", "c"]},
    ]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(name), "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = CONFIGS[name]["vocab"]
    want = {"a": plain_logits(name, 40, 1), "b": plain_logits(name, 9, 2), "c": plain_logits(name, 30, 3)}
    rows = {0: [("a", 0), ("a", 32)], 1: [("a", 33), ("b", 8)], 3: [("c", 29), ("a", 39)]}
    assert not (out / "2.f32").exists()
    for step, places in rows.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape[0] == len(places)
        for r, (rid, p) in enumerate(places):
            close(got[r], want[rid][p], F32_TOL)
    cli = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmx"), "logits", model_folder(name), " ".join(map(str, b)), "--dtype", "f32", "--top", "1"],
                         capture_output=True, text=True, timeout=600)
    assert cli.returncode == 0, cli.stderr[-2000:]
    assert int(cli.stdout.splitlines()[-1].split()[0]) == int(torch.argmax(want["b"][8]))


def test_command_line_generates_from_a_configuration_with_random_weights(tmp_path):
    """`llmx generate --config JSON --random SEED` for this design: weights generated on the device, the scheduler's loop,
    the device sampler."""
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIGS["A"]))
    outs = []
    for _ in range(2):
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmx"), "generate", "--config", str(cfg), "--random", "5", "--std", "0.06",
                              "3 1 4 1 5 9 2 6", "-n", "9", "--temp", "0"], capture_output=True, text=True, timeout=600)
        assert run.returncode == 0, run.stderr[-2000:]
        ids = [int(t) for t in run.stdout.split()]
        assert len(ids) == 9 and all(0 <= t < CONFIGS["A"]["vocab"] for t in ids)
        outs.append(ids)
    assert outs[0] == outs[1]
