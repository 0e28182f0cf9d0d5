"""Causal grouped-query softmax attention over the paged cache.

Per row: q, k, v projections of the normed input (biases optional); an optional RMSNorm over the whole q and the whole k
projection, or over every q and k head by itself with one weight of head_dim values for all heads; rotation of the first `rotary_dim` values of each head at the row's position; k and v written to the
request's pages; softmax(q.k * head_dim^-1/2) over keys 0..p (or the last `window`) of the same request, head h reading
KV head h / (heads / kv_heads); output projection.  Formula order: /root/reference/src/backends/cpu/cpu_backend.hpp:971-1104
(attention), :1461-1480 (rotation); the norm over the whole projection is this architecture's variant of the
reference's per-head norm (/root/reference/src/model/arch/minimax_m3.hpp:258-259).
"""

from __future__ import annotations

import numpy as np
import torch

from .. import ops
from ..limits import MAX_HEAD_DIM
from .base import BuildContext, LayerCache, Mixer, build_part, register
from .spec import CacheTensor, KVNeed, PagedNeed, PartSpec, TensorSpec

_NORM_MODES = {"none": ops.QKNORM_NONE, "projection": ops.QKNORM_PROJECTION, "head": ops.QKNORM_HEAD}

# the names of an attention's tensors below its prefix; `names` in the parameters replaces any of them
_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "q_norm": "q_norm.weight",
          "k_norm": "k_norm.weight", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
          "head_temperature": "head_temperature", "head_gate": "gate_proj.weight", "output_gate": "out_gate_proj.weight", "sink": "sink",
          "lambda_q1": "lambda_q1", "lambda_k1": "lambda_k1", "lambda_q2": "lambda_q2", "lambda_k2": "lambda_k2"}


def power_slopes(heads: int):
    """slope_h = 2^(-8 (h + 1) / heads) for head h = 0 .. heads - 1: the penalty a head puts on a key's distance."""
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


class Attention(Mixer):
    """params: hidden, heads, kv_heads, head_dim, qk_norm ("projection" | "head" | "none"), eps, window (None | int), position (PartSpec),
    scale (None: head_dim^-1/2; else the factor the scores are multiplied by), v_dim (a value head's width, head_dim by
    default), bias (True: q, k, v and the output projection have biases; "qkv": q, k and v only), head_temperature (True: a
    learned factor a query head on its scores, tensor [heads]; it is folded into the rotated query), head_gate (True: the
    result of head h is multiplied by sigmoid(W_g x)_h, W_g [heads, hidden] reading the mixer's input; its rows ride in the
    fused projection behind v), names ({role: name below the prefix}).
    Further rules, all of which the universal attention kernel carries out: keep_first (with a window: the request's first
    keys stay visible at their true positions, and their pages are kept), chunk (a row sees the keys of its own chunk of
    `chunk` positions, counted from the request's start; earlier chunks' pages are given back), softcap (score <- softcap
    tanh(score / softcap)), distance_slopes (True: slope_h (i - j) is taken off the score of key j for the row at i,
    slope_h = 2^(-8 (h + 1) / heads)), sink (True: a learned logit a head, tensor [heads], in the softmax's denominator
    only), values ("keys": there is no value projection, a value head is its key head as projected, before norm and
    rotation), value_norm (True: a value head is divided by its root mean square, eps inside the root, before it is
    cached), output_gate (True: the concatenated heads are multiplied value by value with sigmoid(W_g x), W_g [heads *
    v_dim, hidden]), difference ({diff}: two score maps a head, [map 1 | map 2] in q's and k's rows and each normed and
    rotated by itself, over one set of values: o = a1 - lambda a2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff from
    four learned vectors [head_dim], then o / rms(o) * (1 - diff) a head)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden = int(p["hidden"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.eps = float(p.get("eps", 0.0))
        self.window = p.get("window")
        if self.heads % self.kv_heads:
            raise ValueError("the head count must be divisible by the KV head count")
        if not 0 < self.head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"attention: head_dim {self.head_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        if p.get("qk_norm", "none") not in _NORM_MODES:
            raise ValueError(f"qk_norm {p.get('qk_norm')!r} is not one of {sorted(_NORM_MODES)}")
        self.norm_mode = _NORM_MODES[p.get("qk_norm", "none")]
        self.position = build_part("position", p.get("position") or PartSpec("none"), ctx)
        pairing = getattr(self.position, "pairing", "halves")
        if pairing not in ("halves", "interleaved"):
            raise ValueError(f"attention: rotary pairing {pairing!r} is not one the kernels rotate (halves, interleaved)")
        self.pairing = ops.ROPE_INTERLEAVED if pairing == "interleaved" else ops.ROPE_HALVES
        # softmax(q.k * scale): head_dim^-1/2 unless the architecture gives its own
        self.scale = float(p["scale"]) if p.get("scale") is not None else float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim)))
        if not self.scale > 0.0:
            raise ValueError(f"attention: the softmax scale must be positive, not {self.scale}")
        self.v_dim = int(p["v_dim"]) if p.get("v_dim") is not None else self.head_dim
        if not 0 < self.v_dim <= MAX_HEAD_DIM:
            raise ValueError(f"attention: v_dim {self.v_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        if p.get("bias", False) not in (False, True, "qkv"):
            raise ValueError(f"attention: bias {p.get('bias')!r} is not one of [False, True, 'qkv']")
        self.bias = bool(p.get("bias", False))
        self.out_bias = p.get("bias", False) is True
        self.head_temperature = bool(p.get("head_temperature", False))
        self.head_gate = bool(p.get("head_gate", False))
        self.keep_first = int(p.get("keep_first") or 0)
        self.chunk = int(p.get("chunk") or 0)
        self.softcap = float(p.get("softcap") or 0.0)
        self.distance_slopes = bool(p.get("distance_slopes", False))
        self.sink = bool(p.get("sink", False))
        if p.get("values", "own") not in ("own", "keys"):
            raise ValueError(f"attention: values {p.get('values')!r} is not one of ['keys', 'own']")
        self.values_from_keys = p.get("values", "own") == "keys"
        self.value_norm = bool(p.get("value_norm", False))
        self.output_gate = bool(p.get("output_gate", False))
        self.difference = dict(p["difference"]) if p.get("difference") else None
        self.maps = 2 if self.difference else 1
        self.diff = float(self.difference["diff"]) if self.difference else 0.0
        if self.keep_first < 0 or self.chunk < 0 or self.softcap < 0.0 or (self.keep_first and not self.window) or (self.chunk and self.window):
            raise ValueError("attention: keep_first goes with a window, a chunk without one, and neither they nor softcap are negative")
        if self.values_from_keys and self.v_dim != self.head_dim:
            raise ValueError("attention: values taken from the keys are as wide as the keys")
        if self.output_gate and self.head_gate:
            raise ValueError("attention: a gate a head or a gate a value, not both")
        if self.difference and (self.head_gate or self.head_temperature):
            raise ValueError("attention: two score maps a head go without a gate or temperature a head")
        # what only the universal kernel carries out
        self.special = bool(self.keep_first or self.chunk or self.softcap or self.distance_slopes or self.sink or self.values_from_keys
                            or self.value_norm or self.output_gate or self.difference)
        self.names = dict(_NAMES)
        unknown = set(p.get("names") or {}) - set(_NAMES)
        if unknown:
            raise ValueError(f"attention: no tensor role named {sorted(unknown)}")
        self.names.update(p.get("names") or {})
        self.q_width = self.heads * self.maps * self.head_dim
        self.kv_width = self.kv_heads * self.maps * self.head_dim
        self.v_width = 0 if self.values_from_keys else self.kv_heads * self.v_dim
        self.o_width = self.heads * self.v_dim
        # the plain case (one width, no biases, no norm a head) keeps the kernel that norms whole projections
        self.by_head = (self.norm_mode == ops.QKNORM_HEAD or self.bias or self.v_dim != self.head_dim or self.head_temperature
                        or self.head_gate or self.special)
        self.gate_width = self.heads if self.head_gate else self.o_width if self.output_gate else 0
        if self.by_head and self.norm_mode == ops.QKNORM_PROJECTION:
            raise ValueError("attention: a norm over the whole projection goes with values as wide as keys and no biases")
        self.wqkv = self.wo = self.q_norm = self.k_norm = self.b_qkv = self.b_o = self.temperature = None
        self.sink_logits = self.slopes = self.rules = None
        self.lam = 0.0
        if self.distance_slopes:
            self.slopes = torch.tensor(power_slopes(self.heads), dtype=torch.float64).to(torch.float32).to(ctx.device)

    def cache_need(self):
        if self.v_dim == self.head_dim and not self.special:
            return KVNeed(self.kv_heads, self.head_dim, self.window)
        return PagedNeed((CacheTensor("k", (self.kv_heads * self.maps, self.head_dim), None, 1), CacheTensor("v", (self.kv_heads, self.v_dim), None, 2)),
                         self.window, self.keep_first, self.chunk or None)

    def tensor(self, role):
        return self.name(self.names[role])

    def tensor_specs(self, available):
        # one product for the three projections: the file's q, k and v go straight into the rows q | k | v of one tensor
        q, kv, vw = self.q_width, self.kv_width, self.v_width
        fused, shape = self.name("qkv_proj.weight"), (q + kv + vw + self.gate_width, self.hidden)
        specs = [
            TensorSpec(self.tensor("q"), (q, self.hidden), into=(fused, shape, (slice(0, q),))),
            TensorSpec(self.tensor("k"), (kv, self.hidden), into=(fused, shape, (slice(q, q + kv),))),
            TensorSpec(self.tensor("o"), (self.hidden, self.o_width)),
        ]
        if not self.values_from_keys:
            specs.insert(2, TensorSpec(self.tensor("v"), (vw, self.hidden), into=(fused, shape, (slice(q + kv, q + kv + vw),))))
        if self.norm_mode == ops.QKNORM_PROJECTION:
            specs += [TensorSpec(self.tensor("q_norm"), (q,), "norm"), TensorSpec(self.tensor("k_norm"), (kv,), "norm")]
        elif self.norm_mode == ops.QKNORM_HEAD:
            specs += [TensorSpec(self.tensor("q_norm"), (self.head_dim,), "norm"), TensorSpec(self.tensor("k_norm"), (self.head_dim,), "norm")]
        if self.bias:
            fused_b, shape_b = self.name("qkv_proj.bias"), (q + kv + vw,)
            specs += [TensorSpec(self.tensor("q_bias"), (q,), "bias", into=(fused_b, shape_b, (slice(0, q),))),
                      TensorSpec(self.tensor("k_bias"), (kv,), "bias", into=(fused_b, shape_b, (slice(q, q + kv),))),
                      TensorSpec(self.tensor("v_bias"), (vw,), "bias", into=(fused_b, shape_b, (slice(q + kv, q + kv + vw),)))]
            if self.out_bias:
                specs.append(TensorSpec(self.tensor("o_bias"), (self.hidden,), "bias"))
        if self.head_gate:
            specs.append(TensorSpec(self.tensor("head_gate"), (self.heads, self.hidden), into=(fused, shape, (slice(q + kv + vw, q + kv + vw + self.heads),))))
        if self.output_gate:
            specs.append(TensorSpec(self.tensor("output_gate"), (self.o_width, self.hidden), into=(fused, shape, (slice(q + kv + vw, q + kv + vw + self.o_width),))))
        if self.head_temperature:
            specs.append(TensorSpec(self.tensor("head_temperature"), (self.heads,), "bias", dtype="float32", init=("uniform", 0.5, 1.5)))
        if self.sink:
            specs.append(TensorSpec(self.tensor("sink"), (self.heads,), "bias", dtype="float32", init=("uniform", -1.0, 1.0)))
        if self.difference:
            specs += [TensorSpec(self.tensor(r), (self.head_dim,), "bias", dtype="float32", init=("uniform", -0.3, 0.3))
                      for r in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2")]
        return specs

    def load(self, tensors):
        self.wqkv = tensors[self.name("qkv_proj.weight")]
        self.wo = tensors[self.tensor("o")]
        if self.norm_mode != ops.QKNORM_NONE:
            self.q_norm = tensors[self.tensor("q_norm")]
            self.k_norm = tensors[self.tensor("k_norm")]
        if self.bias:
            self.b_qkv = tensors[self.name("qkv_proj.bias")]
            if self.out_bias:
                self.b_o = tensors[self.tensor("o_bias")]
        if self.head_temperature:
            self.temperature = tensors[self.tensor("head_temperature")]
        if self.sink:
            self.sink_logits = tensors[self.tensor("sink")]
        if self.difference:
            # one number for the layer, formed once from the four vectors
            lq1, lk1, lq2, lk2 = (tensors[self.tensor(r)].to(torch.float64) for r in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2"))
            self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())) + self.diff
        if self.special:
            self.rules = ops.ScoreRules(self.keep_first, self.chunk, self.softcap, self.slopes, self.sink_logits, self.maps)

    def output_bias(self):
        """The output projection's bias, which a caller that joins this mixer's result with others may add itself
        (forward(..., add_output_bias=False)); None without one."""
        return self.b_o

    def takes_deferred_norm(self, step):
        return ops.gemm_takes_normed_rows(step.rows, self.wqkv, torch.float32)

    def _plan(self, step):
        """The matrix-core attention kernel's work items for this step's rows: made once a step and shared by every
        layer with the same heads and window."""
        window = int(self.window or 0)
        return step.shared(("attention.plan", self.heads, self.kv_heads, window),
                           lambda: ops.attention_plan([e.n for e in step.entries], [e.past + e.n for e in step.entries], self.heads,
                                                      self.kv_heads, step.device, window))

    def _rules_plan(self, step):
        """The work items of the matrix-core kernel for rules, made once a step and shared by every layer with the same
        columns and rules."""
        window = int(self.window or 0)
        shared = ops.attention_rules_shared_ok(self.head_dim, self.v_dim)
        return step.shared(("attention.rules_plan", self.heads, self.kv_heads, self.maps, window, self.keep_first, self.chunk, shared),
                           lambda: ops.rules_plan([e.n for e in step.entries], [e.past + e.n for e in step.entries], self.heads, self.kv_heads,
                                                  self.maps, step.device, window, self.keep_first, self.chunk, shared=shared))

    def _rules_mfma(self, act, page_tokens):
        return self.special and ops.attention_rules_ok(act, self.head_dim, self.v_dim, page_tokens)

    def graph_key(self, step):
        # a recorded step holds the plan's addresses and launch sizes; the universal kernel has no plan
        page = self.ctx.page_tokens
        if page and self._rules_mfma(step.act_dtype, page):
            return self._rules_plan(step)
        return self._plan(step) if page and self._mfma(step.act_dtype, page) else None

    def _mfma(self, act, page_tokens):
        return self.v_dim == self.head_dim and not self.special and ops.attention_mfma_ok(act, self.head_dim, page_tokens)

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None, add_output_bias=True):
        T = step.rows
        act = step.act_dtype
        qkv_width = self.q_width + self.kv_width + self.v_width
        qkv = step.buf("attention.qkv", (T, qkv_width + self.gate_width), torch.float32)
        ops.gemm(h, self.wqkv, qkv, scratch=step.buf)
        q = step.buf("attention.q", (T, self.q_width), act)
        cos_sin, rotary = self.position.rotation()
        tables = step.tables(cache.group)
        if self.by_head:
            ops.head_norm_rope_kvwrite(qkv, self.b_qkv, self.q_norm, self.k_norm, cos_sin, step.positions, step.row_entry, tables, q, cache.k,
                                       cache.v, self.eps, self.heads, self.kv_heads, self.head_dim, rotary, self.norm_mode,
                                       write_kv=cache.writes, pairing=self.pairing, q_scale=self.temperature, maps=self.maps,
                                       values_from_keys=self.values_from_keys, value_norm=self.value_norm)
        else:
            ops.qknorm_rope_kvwrite(qkv, self.q_norm, self.k_norm, cos_sin, step.positions, step.row_entry, tables, q, cache.k, cache.v,
                                    self.eps, self.heads, self.kv_heads, self.head_dim, rotary, self.norm_mode, write_kv=cache.writes,
                                    pairing=self.pairing)
        o = step.buf("attention.out", (T, self.o_width), act)
        plan = self._plan(step) if self._mfma(act, cache.k.shape[2]) else None
        by_rules = self._rules_plan(step) if self._rules_mfma(act, cache.k.shape[2]) else None
        if self.difference:
            # both maps' results in float32, then their difference, its norm a head and the gate in one kernel
            both = step.buf("attention.maps", (T, self.maps * self.o_width), torch.float32)
            ops.paged_attention(q, cache.k, cache.v, step.positions, step.row_entry, tables, both, self.scale, self.heads,
                                window=int(self.window or 0), rules=self.rules, rules_plan=by_rules, scratch=step.buf)
            ops.head_norm_gate(both, None, qkv[:, qkv_width:] if self.output_gate else None, o, self.eps, self.heads, self.v_dim,
                               ops.GATE_SIGMOID, minus=self.lam, post=1.0 - self.diff)
        else:
            ops.paged_attention(q, cache.k, cache.v, step.positions, step.row_entry, tables, o, self.scale, self.heads,
                                window=int(self.window or 0), plan=plan, scratch=step.buf,
                                head_gate=qkv[:, qkv_width:] if self.head_gate else None,      # the gate a head, where the result is stored
                                rules=self.rules, output_gate=qkv[:, qkv_width:] if self.output_gate else None, rules_plan=by_rules)
        if self.b_o is not None and add_output_bias:
            y = step.buf("attention.projected", (T, self.hidden), torch.float32)
            ops.gemm(o, self.wo, y, scratch=step.buf)
            ops.combine_rows(out, y, 1.0, self.b_o, accumulate=accumulate)
        else:
            ops.gemm(o, self.wo, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "attention", Attention)
