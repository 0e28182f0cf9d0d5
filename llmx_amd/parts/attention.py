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
          "head_temperature": "head_temperature", "head_gate": "gate_proj.weight"}


class Attention(Mixer):
    """params: hidden, heads, kv_heads, head_dim, qk_norm ("projection" | "head" | "none"), eps, window (None | int), position (PartSpec),
    scale (None: head_dim^-1/2; else the factor the scores are multiplied by), v_dim (a value head's width, head_dim by
    default), bias (True: q, k, v and the output projection have biases; "qkv": q, k and v only), head_temperature (True: a
    learned factor a query head on its scores, tensor [heads]; it is folded into the rotated query), head_gate (True: the
    result of head h is multiplied by sigmoid(W_g x)_h, W_g [heads, hidden] reading the mixer's input; its rows ride in the
    fused projection behind v), names ({role: name below the prefix})."""
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
        self.names = dict(_NAMES)
        unknown = set(p.get("names") or {}) - set(_NAMES)
        if unknown:
            raise ValueError(f"attention: no tensor role named {sorted(unknown)}")
        self.names.update(p.get("names") or {})
        self.q_width = self.heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.v_width = self.kv_heads * self.v_dim
        self.o_width = self.heads * self.v_dim
        # the plain case (one width, no biases, no norm a head) keeps the kernel that norms whole projections
        self.by_head = (self.norm_mode == ops.QKNORM_HEAD or self.bias or self.v_dim != self.head_dim or self.head_temperature
                        or self.head_gate)
        self.gate_width = self.heads if self.head_gate else 0
        if self.by_head and self.norm_mode == ops.QKNORM_PROJECTION:
            raise ValueError("attention: a norm over the whole projection goes with values as wide as keys and no biases")
        self.wqkv = self.wo = self.q_norm = self.k_norm = self.b_qkv = self.b_o = self.temperature = None

    def cache_need(self):
        if self.v_dim == self.head_dim:
            return KVNeed(self.kv_heads, self.head_dim, self.window)
        return PagedNeed((CacheTensor("k", (self.kv_heads, self.head_dim), None, 1), CacheTensor("v", (self.kv_heads, self.v_dim), None, 2)),
                         self.window)

    def tensor(self, role):
        return self.name(self.names[role])

    def tensor_specs(self, available):
        # one product for the three projections: the file's q, k and v go straight into the rows q | k | v of one tensor
        q, kv, vw = self.q_width, self.kv_width, self.v_width
        fused, shape = self.name("qkv_proj.weight"), (q + kv + vw + self.gate_width, self.hidden)
        specs = [
            TensorSpec(self.tensor("q"), (q, self.hidden), into=(fused, shape, (slice(0, q),))),
            TensorSpec(self.tensor("k"), (kv, self.hidden), into=(fused, shape, (slice(q, q + kv),))),
            TensorSpec(self.tensor("v"), (vw, self.hidden), into=(fused, shape, (slice(q + kv, q + kv + vw),))),
            TensorSpec(self.tensor("o"), (self.hidden, self.o_width)),
        ]
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
        if self.head_temperature:
            specs.append(TensorSpec(self.tensor("head_temperature"), (self.heads,), "bias", dtype="float32", init=("uniform", 0.5, 1.5)))
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

    def graph_key(self, step):
        # a recorded step holds the plan's addresses and launch sizes; the universal kernel has no plan
        page = self.ctx.page_tokens
        return self._plan(step) if page and self._mfma(step.act_dtype, page) else None

    def _mfma(self, act, page_tokens):
        return self.v_dim == self.head_dim and ops.attention_mfma_ok(act, self.head_dim, page_tokens)

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
                                       write_kv=cache.writes, pairing=self.pairing, q_scale=self.temperature)
        else:
            ops.qknorm_rope_kvwrite(qkv, self.q_norm, self.k_norm, cos_sin, step.positions, step.row_entry, tables, q, cache.k, cache.v,
                                    self.eps, self.heads, self.kv_heads, self.head_dim, rotary, self.norm_mode, write_kv=cache.writes,
                                    pairing=self.pairing)
        o = step.buf("attention.out", (T, self.o_width), act)
        plan = self._plan(step) if self._mfma(act, cache.k.shape[2]) else None
        ops.paged_attention(q, cache.k, cache.v, step.positions, step.row_entry, tables, o, self.scale, self.heads,
                            window=int(self.window or 0), plan=plan, scratch=step.buf,
                            head_gate=qkv[:, qkv_width:] if self.head_gate else None)      # the gate a head, where the result is stored
        if self.b_o is not None and add_output_bias:
            y = step.buf("attention.projected", (T, self.hidden), torch.float32)
            ops.gemm(o, self.wo, y, scratch=step.buf)
            ops.combine_rows(out, y, 1.0, self.b_o, accumulate=accumulate)
        else:
            ops.gemm(o, self.wo, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "attention", Attention)
