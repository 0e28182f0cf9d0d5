"""Salipel in the engine against the plain implementation (tests/plain_salipel.py), mechanism by mechanism and whole.

Kernels alone (the gated units in the products' epilogues, the three attention forms over shuffled pages with one query made
to fit a single key on both sides of every edge: a window's, the kept first tokens', a chunk's, a page's; the matrix memory
through its preparation, the scan and the read-out, carried over cuts) against the plain functions; then the engine under
every way of cutting the same tokens into steps, which must agree bit for bit with each other in both dtypes, with the
plain implementation within F32_TOL in float32 and within BF16_TOL in bfloat16 (the engine's expert picks handed over);
pages and request seats that are used again; long decoding past windows and chunks; greedy generation through `generate`;
the trace replay tool and the command line.
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

import plain_salipel as plain
from salipel_cases import CONFIGS, PAGES, greedy, load_plain, model_folder, plain_logits, portions, routed_layers, tokens_for, write_folder

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # |engine - plain| over all logits relative to the largest |logit|: float32 sums in another order
BF16_TOL = 6e-2     # the serving path against the plain implementation (float64, nothing rounded), with the engine's expert picks
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
# kernels alone: the units
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 3, 40, 300])
def test_products_with_the_gelu_gate_and_the_squared_relu(dtype, rows):
    """Dense gate_up with gelu_tanh(gate) * up in the epilogue and grouped up-products with max(z, 0)^2, at row counts that
    take the weight-streaming, the tiled and (float32) the universal kernels."""
    o = ops()
    rng = np.random.default_rng(rows)
    K, F, X, k = 64, 48, 5, 2
    h = rng.normal(size=(rows, K))
    wg = rng.normal(size=(2 * F, K)) * 0.3
    hd, wd = dev(h, dtype), dev(wg, dtype)
    hr, wr = hd.double().cpu().numpy(), wd.double().cpu().numpy()
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    out = torch.empty(rows, F, device="cuda", dtype=dtype)
    o.gemm(hd, wd, out, o.EPI_SWIGLU, glu=o.Glu(o.GLU_GELU_TANH))
    close(out.float(), plain.gelu_tanh(hr @ wr[:F].T) * (hr @ wr[F:].T), tol, "gelu gate")
    # grouped: pairs sorted by expert
    we = rng.normal(size=(X, F, K)) * 0.3
    wed = dev(we, dtype)
    ids = np.stack([rng.permutation(X)[:k] for _ in range(rows)]).astype(np.int32)
    idd = dev(ids, torch.int32)
    counts, offsets = torch.empty(X, device="cuda", dtype=torch.int32), torch.empty(X + 1, device="cuda", dtype=torch.int32)
    pairs, active, n_active = (torch.empty(n, device="cuda", dtype=torch.int32) for n in (rows * k, X, 1))
    o.moe_align(idd, X, counts, offsets, pairs, active, n_active)
    act = torch.zeros(rows * k, F, device="cuda", dtype=dtype)
    o.grouped_gemm(hd, wed, act, offsets, pairs, k, o.EPI_STORE, active, n_active, token_rows=rows, act=(o.ACT_RELU2, None))
    wer = wed.double().cpu().numpy()
    want = np.stack([np.maximum(wer[ids[t, j]] @ hr[t], 0.0) ** 2 for t in range(rows) for j in range(k)])
    close(act.float(), want, tol, "squared relu, grouped")
    plainly = torch.empty(rows, F, device="cuda", dtype=dtype)
    o.gemm(hd, wed[0].contiguous(), plainly, act=(o.ACT_RELU2, None))
    close(plainly.float(), np.maximum(hr @ wer[0].T, 0.0) ** 2, tol, "squared relu, dense")


# ---------------------------------------------------------------------------
# kernels alone: attention
def _attention_weights(rng, kind, E, H, G, D, V):
    M = 2 if kind == "two_maps" else 1
    W = {"p.q": rng.normal(size=(H * M * D, E)) * 0.5, "p.k": rng.normal(size=(G * M * D, E)) * 0.5, "p.o": np.eye(H * V)}
    if kind != "window":
        W["p.v"] = rng.normal(size=(G * V, E)) * 0.5
    if kind != "chunks":
        W.update({"p.q.norm": rng.uniform(0.5, 1.5, size=D), "p.k.norm": rng.uniform(0.5, 1.5, size=D), "p.g": rng.normal(size=(H * V, E)) * 0.5})
    if kind == "chunks":
        W["p.sink"] = rng.normal(size=H)
    if kind == "two_maps":
        W.update({n: rng.normal(size=D) * 0.3 for n in ("p.lq1", "p.lk1", "p.lq2", "p.lk2")})
    return W


def _attention_case(dtype, kind, H, G, D, V, R, page, length, rule, sharp=None, decode_from=None, scale=0.3, scaling=None, shared=True):
    """One attention part alone through its kernels (the step before the attention, the attention over shuffled pages, the
    join of two maps) against the plain mixer.  kind: "window" (rule = (size, keep_first)), "chunks" (rule = size) or
    "two_maps" (rule = (softcap, diff)).  sharp = (row, key): the row's query is made to fit that key alone, whether the
    row may see it or not.  decode_from: rows from there on are run one by one, each in launches of its own."""
    from llmx_amd.parts.attention import power_slopes
    from llmx_amd.parts.position import scaled_table
    rng = np.random.default_rng(H * 1000 + D + length)
    o = ops()
    E = 24
    M = 2 if kind == "two_maps" else 1
    W = _attention_weights(rng, kind, E, H, G, D, V)
    h = rng.normal(size=(length, E))
    if sharp is not None:
        # the key row's input is far from all others and the query row's input is the same; every query head is made the
        # key head's projection, so that key's score stands out as far as norm and rotation let it
        row, key = sharp
        h[key] = h[key] * 5
        h[row] = h[key]
        W["p.q"] = np.concatenate([W["p.k"].reshape(G, M * D, E)[hh // (H // G)] for hh in range(H)]) * (4.0 if kind == "chunks" else 1.0)
        if kind != "chunks":
            W["p.q.norm"] = W["p.k.norm"] * 6.0
    sc = dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None
    rot = {"base": 500.0, "dims": R, "scaling": sc}
    eps = 1e-6
    if kind == "window":
        cfg = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "mask": {"size": rule[0], "keep_first": rule[1]}, "rot": rot}
        want = plain.window_attention(h, W, "p.", cfg, eps)
        rules = o.ScoreRules(keep_first=rule[1])
        window = rule[0]
    elif kind == "chunks":
        cfg = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "mask": {"size": rule}}
        want = plain.chunk_attention(h, W, "p.", cfg, eps)
        rules = o.ScoreRules(chunk=rule, slopes=dev(np.asarray(power_slopes(H))), sink=dev(W["p.sink"]))
        window = 0
    else:
        cfg = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "softcap": rule[0], "diff": rule[1], "rot": rot}
        want = plain.difference_attention(h, W, "p.", cfg, eps)
        rules = o.ScoreRules(softcap=rule[0] or 0.0, maps=2)
        window = 0
    cols = [h @ W["p.q"].T, h @ W["p.k"].T] + ([h @ W["p.v"].T] if kind != "window" else []) + ([h @ W["p.g"].T] if kind != "chunks" else [])
    proj = np.concatenate(cols, axis=1)
    width = H * M * D + G * M * D + (0 if kind == "window" else G * V)
    n_pages = -(-length // page)
    order = list(range(n_pages + 3))
    random.Random(length).shuffle(order)
    tables = dev(np.array([order[:n_pages] + [-1] * 5]), torch.int32)
    kc = torch.zeros(n_pages + 3, G * M, page, D, device="cuda", dtype=dtype)
    vc = torch.zeros(n_pages + 3, G, V, page, device="cuda", dtype=dtype)
    cos_sin = dev(scaled_table(length, R, 500.0, sc))
    normed = kind != "chunks"
    qw, kw = (dev(W["p.q.norm"]), dev(W["p.k.norm"])) if normed else (None, None)
    out = torch.empty(length, H * V, device="cuda", dtype=dtype)
    runs = [(0, length)] if decode_from is None else [(0, decode_from)] + [(i, i + 1) for i in range(decode_from, length)]
    for a, b in runs:
        n = b - a
        pos, ent = dev(np.arange(a, b), torch.int32), dev(np.zeros(n), torch.int32)
        rows = dev(proj[a:b])
        q = torch.empty(n, H * M * D, device="cuda", dtype=dtype)
        o.head_norm_rope_kvwrite(rows, None, qw, kw, cos_sin, pos, ent, tables, q, kc, vc, eps, H, G, D, R, o.QKNORM_HEAD if normed else o.QKNORM_NONE,
                                 pairing=o.ROPE_HALVES, maps=M, values_from_keys=kind == "window", value_norm=kind == "chunks")
        part = torch.empty(n, H * V, device="cuda", dtype=dtype)
        # where the sizes allow, the matrix-core kernel for rules (its work items made for this launch's rows)
        plan = None
        if o.attention_rules_ok(dtype, D, V, page):
            plan = o.rules_plan([n], [b], H, G, M, torch.device("cuda"), window, rules.keep_first, rules.chunk,
                                shared=shared and o.attention_rules_shared_ok(D, V))
        if kind == "two_maps":
            both = torch.empty(n, H * 2 * V, device="cuda", dtype=torch.float32)
            o.paged_attention(q, kc, vc, pos, ent, tables, both, scale, H, rules=rules, rules_plan=plan)
            o.head_norm_gate(both, None, rows[:, width:], part, eps, H, V, o.GATE_SIGMOID, minus=plain.difference_lambda(W, "p.", rule[1]), post=1.0 - rule[1])
        else:
            o.paged_attention(q, kc, vc, pos, ent, tables, part, scale, H, window=window, rules=rules,
                              output_gate=rows[:, width:] if kind == "window" else None, rules_plan=plan)
        out[a:b] = part
    return out.float().cpu(), torch.as_tensor(want)


ATT_TOL = {torch.float32: 2e-5, torch.bfloat16: 4e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [
    ("window", 4, 2, 32, 32, 16, 16, 150, (24, 3)), ("window", 3, 1, 10, 10, 6, 4, 90, (5, 0)), ("window", 2, 2, 128, 128, 64, 16, 200, (70, 9)),
    ("window", 4, 4, 16, 16, 16, 16, 60, (300, 8)), ("window", 2, 1, 24, 24, 0, 8, 70, (1, 5)), ("window", 2, 1, 64, 64, 32, 16, 1300, (700, 300)),
    ("chunks", 4, 1, 16, 32, 0, 16, 150, 40), ("chunks", 3, 3, 10, 6, 0, 4, 60, 7), ("chunks", 8, 2, 64, 64, 0, 16, 200, 64), ("chunks", 2, 1, 48, 8, 0, 16, 40, 1),
    ("two_maps", 4, 2, 32, 64, 16, 16, 150, (30.0, 0.25)), ("two_maps", 3, 1, 10, 14, 10, 4, 70, (1.5, 0.5)), ("two_maps", 2, 2, 64, 128, 0, 16, 130, (None, 0.3)),
    ("two_maps", 2, 1, 48, 96, 16, 16, 1100, (20.0, 0.2)), ("chunks", 2, 1, 32, 48, 0, 16, 1200, 600),
    # the widest heads the kernels take, sixteen query heads a key head, the narrowest the matrix cores take, kept tokens over
    # several segments beside a short window, a chunk that is no multiple of anything
    ("window", 2, 1, 256, 256, 64, 16, 300, (90, 10)), ("two_maps", 1, 1, 256, 256, 32, 16, 200, (15.0, 0.1)), ("chunks", 16, 1, 8, 16, 0, 16, 180, 33),
    ("window", 16, 1, 16, 16, 8, 32, 700, (40, 300)), ("two_maps", 5, 1, 24, 256, 8, 16, 160, (5.0, 0.4)), ("chunks", 4, 2, 256, 64, 0, 48, 400, 129),
    ("window", 8, 1, 128, 128, 128, 16, 260, (17, 1)),
], ids=lambda c: f"{c[0]}-{c[1]}x{c[3]}")
def test_the_three_attention_forms_over_shuffled_pages(dtype, case):
    kind, H, G, D, V, R, page, length, rule = case
    scaling = (4.0, 1.0, 4.0, 64) if R >= 16 else None
    scale = 0.3 * min(1.0, (64.0 / D) ** 0.5)       # wide heads' scores stay of a size at which bfloat16 keys do not decide the softmax
    got, want = _attention_case(dtype, kind, H, G, D, V, R, page, length, rule, scaling=scaling, scale=scale)
    close(got, want, ATT_TOL[dtype], "a prompt")
    decoded, want = _attention_case(dtype, kind, H, G, D, V, R, page, length, rule, decode_from=length - 30, scaling=scaling, scale=scale)
    close(decoded, want, ATT_TOL[dtype], "a decoded tail")
    # the four-wave form, the one-wave form and rows decoded alone give a row the same bits
    alone, _ = _attention_case(dtype, kind, H, G, D, V, R, page, length, rule, scaling=scaling, shared=False, scale=scale)
    assert torch.equal(alone, got) and torch.equal(decoded, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [False, True], ids=["prompt", "decoded"])
def test_one_key_on_both_sides_of_every_edge(dtype, decoded):
    """The last row's query fits one key: just inside and just outside the window, the last kept token and the first one
    not kept, the first and the last key of the row's chunk and the last of the chunk before, keys at page borders, the
    first token, the row itself, and for the causal form keys hundreds of rows back."""
    length = 260
    row = length - 1
    size, keep = 72 + 5, 4
    for key in (0, 1, keep - 1, keep, keep + 1, 15, 16, row - size - 1, row - size, row - size + 1, row - size + 2, row - 1, row):
        got, want = _attention_case(dtype, "window", 2, 1, 32, 32, 16, 16, length, (size, keep), sharp=(row, key), decode_from=row - 3 if decoded else None)
        close(got[row], want[row], ATT_TOL[dtype] * 2, f"window, key {key}")
    chunk = 50
    start = (row // chunk) * chunk
    for key in (0, start - 2, start - 1, start, start + 1, 255, 256, row):
        got, want = _attention_case(dtype, "chunks", 4, 2, 16, 24, 0, 16, length, chunk, sharp=(row, key), decode_from=row - 3 if decoded else None, scale=0.5)
        close(got[row], want[row], ATT_TOL[dtype] * 2, f"chunks, key {key}")
    for key in (0, 1, 15, 16, 63, 64, 65, 127, 128, 200, row - 1):
        got, want = _attention_case(dtype, "two_maps", 2, 1, 32, 48, 16, 16, length, (40.0, 0.3), sharp=(row, key), decode_from=row - 3 if decoded else None)
        close(got[row], want[row], ATT_TOL[dtype] * 2, f"two maps, key {key}")
    # the sharp keys do carry the weight where they are seen, and none where they are not (float64, the plain functions alone)
    if dtype == torch.float32 and not decoded:
        _, inside = _attention_case(dtype, "window", 2, 1, 32, 32, 16, 16, length, (size, keep), sharp=(row, row - size + 1))
        _, outside = _attention_case(dtype, "window", 2, 1, 32, 32, 16, 16, length, (size, keep), sharp=(row, row - size))
        _, kept = _attention_case(dtype, "window", 2, 1, 32, 32, 16, 16, length, (size, keep), sharp=(row, keep - 1))
        assert float((inside[row] - outside[row]).abs().max()) > 0.05 and float((kept[row] - outside[row]).abs().max()) > 0.05


# ---------------------------------------------------------------------------
# kernels alone: the matrix memory
@pytest.mark.parametrize("sizes", [(2, 16, 24), (1, 7, 9), (4, 64, 16), (1, 80, 40), (2, 128, 128), (1, 200, 33)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("gates", [1.0, 6.0], ids=["mild gates", "wide gates"])
def test_matrix_memory_preparation_scan_and_read_out(sizes, gates):
    """Two requests of unequal length in one launch, then carried on in portions and single tokens from their state slots
    (read at one slot, written at another); float32 throughout."""
    o = ops()
    H, D, V = sizes
    rng = np.random.default_rng(D * 7 + V)
    E, cap, eps = 20, 5.0, 1e-6
    cfg = {"heads": H, "dim": D, "vdim": V, "gate_cap": cap}
    W = {"m." + n: rng.normal(size=s) * 0.4 for n, s in (("q", (H * D, E)), ("k", (H * D, E)), ("v", (H * V, E)), ("g", (H * V, E)),
                                                         ("i", (H, E)), ("f", (H, E)))}
    W["m.i"] *= gates
    W["m.f"] *= gates
    W.update({"m.i.b": rng.normal(size=H), "m.f.b": rng.normal(size=H) + 1.0, "m.norm": rng.uniform(0.5, 1.5, size=H * V), "m.o": np.eye(H * V)})
    lengths = [45, 300]
    hs = [rng.normal(size=(n, E)) for n in lengths]
    want = [plain.matrix_memory(h, W, "m.", cfg, eps)[0] for h in hs]
    w_in = np.concatenate([W["m." + n] for n in ("q", "k", "v", "g", "i", "f")])
    HD, HV = H * D, H * V
    cols = {"q": 0, "k": HD, "v": 2 * HD, "g": 2 * HD + HV, "i": 2 * HD + 2 * HV, "f": 2 * HD + 2 * HV + H}
    m_off = o.state_matrix_size(H, D, V + 1)
    state = torch.zeros(4, m_off + H, device="cuda")
    held = [0, 1]
    got = [[], []]
    cuts = [[(0, 45)], [(0, 200), (200, 201), (201, 203), (203, 300)]]
    for step in range(4):
        live = [r for r in range(2) if step < len(cuts[r])]
        parts = [hs[r][cuts[r][step][0]:cuts[r][step][1]] for r in live]
        rows = np.concatenate(parts)
        T = rows.shape[0]
        pre = dev(rows @ w_in.T)
        to = [(held[r] + 2) % 4 for r in live]    # the step writes another slot than it reads: 0 <-> 2, 1 <-> 3
        entry_rows, at = [], 0
        for p in parts:
            entry_rows.append([at, p.shape[0]])
            at += p.shape[0]
        slot_read, slot_write, er = dev([held[r] for r in live], torch.int32), dev(to, torch.int32), dev(entry_rows, torch.int32)
        decay, keys = torch.empty(T, HD, device="cuda"), torch.empty(T, HD, device="cuda")
        values, floor = torch.empty(T, H * (V + 1), device="cuda"), torch.empty(T, H, device="cuda")
        o.memory_prep(pre, cols, dev(W["m.i.b"]), dev(W["m.f.b"]), cap, state, m_off, slot_read, slot_write, er, decay, keys, values, floor, H, D, V)
        out = torch.empty(T, H * (V + 1), device="cuda")
        o.state_scan(pre[:, :HD], keys, values, decay, None, state, slot_read, slot_write, er, out, float(D) ** -0.5, H, H, D, V + 1,
                     max_rows=max(p.shape[0] for p in parts))
        y = torch.empty(T, HV, device="cuda")
        o.head_norm_gate(out, dev(W["m.norm"]), pre[:, cols["g"]:cols["g"] + HV], y, eps, H, V, o.GATE_SIGMOID, den_floor=floor)
        at = 0
        for r, p in zip(live, parts):
            got[r].append(y[at:at + p.shape[0]].cpu())
            at += p.shape[0]
        for r, slot in zip(live, to):
            held[r] = slot
    for r in range(2):
        close(torch.cat(got[r]), want[r], 3e-5, f"request {r}")


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
    """(rows, picks): a whole prompt's logits and, for every routed layer in order, the experts the engine picked [T, top]."""
    shown = []
    engine.observer = lambda step, kind, **t: shown.append(t["ids"].cpu().numpy().copy()) if kind == "routing" else None
    try:
        rows = run_cut(engine, "picks", tokens, [(0, len(tokens))])
    finally:
        engine.observer = None
    return rows, shown


def reference_rows(name, dtype, length, seed, got, engine=None, folder=None, tol=None):
    """float32 against the plain implementation.  bfloat16 too, within BF16_TOL, with the engine's own expert picks handed
    to the plain implementation (a near tie of two choice scores may fall the other way after rounding, and then another
    expert runs); `got` must be the bits of the whole prompt that was run to see the picks."""
    tokens = tokens_for(name, length, seed)
    if dtype == "float32":
        want = plain_logits(name, length, seed) if folder is None else plain.forward(*load_plain(folder), tokens)
        close(got, want, tol or F32_TOL, "against the plain implementation")
        return
    rows, picks = run_whole_with_picks(engine, tokens)
    assert torch.equal(rows, got), "the whole prompt run again gives other bits"
    config, tensors = load_plain(folder or model_folder(name))
    want = torch.as_tensor(plain.forward(config, tensors, tokens, picks=dict(zip(routed_layers(config), picks))))
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
    layers = []
    plain.forward(config, tensors, tokens, layers_out=layers)
    seen = []
    engine.observer = lambda step, kind, **t: seen.append(t["residual"].clone()) if kind == "layer" else None
    try:
        run_cut(engine, "layers", tokens, [(0, 21)])
    finally:
        engine.observer = None
    assert len(seen) == len(layers) == len(config["layers"])
    for i, (got, want) in enumerate(zip(seen, layers)):
        close(got, want, F32_TOL, f"residual after layer {i}")


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
    """A short prompt, then 230 tokens one by one over many pages, past every window and through several chunks: the rows of
    the whole sequence, from an engine that replays decode steps as graphs and from one that does not."""
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


def test_windows_and_chunks_give_pages_back_while_a_request_runs():
    """Pages that no later row reads go back to their pools at every commit, the kept first tokens' pages stay, and what is
    read afterwards is still right: a long prompt in portions in an engine whose windowed pools could not hold it whole."""
    name = "A"
    engine = make_engine(name, "float32", kv_tokens=400)
    length = 390
    tokens = tokens_for(name, length, 6)
    from llmx_amd.engine import StepEntry
    engine.add_request("r")
    rows = []
    for a in range(0, length, 30):
        rows.append(engine.step([StepEntry("r", tokens[a:a + 30], list(range(min(30, length - a))))]).clone().cpu())
    by_window = {(g.window, g.chunk): i for i, g in enumerate(engine.cache.groups)}
    used = {k: engine.cache.pages_in_use(i) for k, i in by_window.items()}
    assert used[(24, None)] <= 4 and used[(None, 40)] <= 3 and used[(None, None)] == -(-length // 16)
    table = engine.cache.table("r", by_window[(24, None)])
    assert table[0] >= 0 and table[1] < 0              # the three kept tokens' page stays, the next one is gone
    engine.end_request("r")
    close(torch.cat(rows), plain_logits(name, length, 6), F32_TOL)


def test_which_kernels_a_serving_step_takes():
    """The launch witness: a bfloat16 step at sizes the matrix cores take (configuration A) runs the design's kernels, the
    matrix-core products and the matrix-core attention for rules (a decoded row's context shared out and merged), never
    the universal ones; a float32 engine runs the universal attention and launches no bfloat16 product."""
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
        for name in ("head_norm_rope_kvwrite", "memory_prep", "state_scan", "head_norm_gate", "combine_rows", "rmsnorm",
                     "moe_combine", "route_topk"):
            assert seen.get(name), f"{dtype}: no launch of {name} ({sorted(seen)})"
        if dtype == "bfloat16":     # the prompt's portion by workgroups of four tiles, the decoded row by items and their merge
            assert seen["attention.rules_shared"] == 4 and seen["attention.rules"] == 4
        else:
            assert seen["attention.generic"] == 2 * 4
        assert seen["memory_prep"] == 2 and seen["state_scan"] == 2
        assert seen["head_norm_gate"] == 2 * 3                  # two layers of two maps and the memory's read-out
        assert seen["combine_rows"] == 2 * (4 + 1)              # every layer's join, and the side-by-side mixer's
        assert seen["rmsnorm"] >= 2 * 4                         # one norm a layer (and the model's, where a step wants rows)
        assert "act.glu" not in seen and "gate_heads" not in seen       # the units run in the products' epilogues
        if dtype == "bfloat16":
            assert not any(n.startswith(("gemm_generic", "attention.generic")) for n in seen), sorted(seen)
            assert seen.get("attention.rules_merge")
            assert any(n.startswith("gemm_skinny") or n.startswith("gemm_tile") for n in seen)
        else:
            assert not any(n.startswith(("gemm_skinny", "gemm_tile", "attention.rules")) for n in seen), sorted(seen)


def test_a_failed_step_leaves_pages_and_states_as_they_were():
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
    """Larger query weights (where q is normed: larger norm weights) and lower sinks let the softmax pick single keys, for
    the causal form hundreds of tokens back, so a key lost at a page's, a window's or a chunk's edge shows.  Whole,
    portions and decoding agree bit for bit, and float32 with the plain model."""
    def edit(tensors):
        for k in tensors:
            if k.endswith("q.norm"):
                tensors[k] = tensors[k] * 4.0
            if k.endswith("mix.q") and k.replace("mix.q", "mix.sink") in tensors:
                tensors[k] = (tensors[k].float() * 6.0).to(tensors[k].dtype)
            if k.endswith("mix.sink"):
                tensors[k] = tensors[k] - 3.0
    folder = write_folder(CONFIGS["A"], 37, str(tmp_path / "sharp"), edit)
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
        want = torch.as_tensor(plain.forward(config, tensors, tokens, picks=dict(zip(routed_layers(config), picks))))
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
    # bfloat16: the tokens are compared with those the same engine gives step by step without scheduler and sampler (every
    # cutting gives a row the same bits): whole prompt, then one token at a time, the largest logit each time
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
