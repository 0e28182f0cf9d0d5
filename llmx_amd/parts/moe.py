"""Feed-forward parts: routed SwiGLU experts behind a scored top-k router, a dense SwiGLU, and a dense layer with one
activation between its two products.

Router: z = h.Wr^T in float32 on unrounded rows (/root/reference/src/backends/backend.hpp:944-947); score sigmoid(z);
the pick key is score + correction bias, k picks, the lowest id on ties; weight = the unbiased score, divided by the
picks' sum when normalizing, times the scale (/root/reference/src/backends/cpu/cpu_backend.hpp:2774-2819).
Experts: a = silu(h.Wg_e^T) * (h.Wu_e^T), y = a.Wd_e^T (:3003-3010); the row's result is sum_j w_j * y_j in slot order
(:2840-2867).  The fused gate_up tensor holds gate rows first (/root/reference/tests/fixture_minimax.py:153-155).
"""

from __future__ import annotations

import re

import torch

from .. import ops
from ..limits import MAX_EXPERTS, MAX_TOP_K
from .base import FeedForward, register
from .spec import TensorSpec

_SCORES = {"sigmoid": ops.SCORE_SIGMOID, "softmax": ops.SCORE_SOFTMAX}

# the names of a routed feed-forward's tensors below its prefix ({e}: the expert's number); `names` in the parameters
# replaces any of them
_EXPERT_NAMES = {"router": "gate.weight", "correction_bias": "gate.e_score_correction_bias", "logit_bias": "gate.bias",
                 "fused_gate_up": "experts.gate_up_proj", "fused_down": "experts.down_proj",
                 "expert_gate": "experts.{e}.gate_proj.weight", "expert_up": "experts.{e}.up_proj.weight",
                 "expert_down": "experts.{e}.down_proj.weight"}
_GLU_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
# a shared expert's tensors below the routed feed-forward's prefix
_EXPERT_NAMES.update({"shared_gate": "shared_expert.gate_proj.weight", "shared_up": "shared_expert.up_proj.weight",
                      "shared_down": "shared_expert.down_proj.weight", "shared_switch": "shared_expert_gate.weight"})
_UNITS = {"swiglu": ops.GLU_SILU, "clamped_glu": ops.GLU_CLAMPED, "geglu_tanh": ops.GLU_GELU_TANH}
# units of one product and an activation instead of two products and a gate
_PLAIN_UNITS = {"relu2": ops.ACT_RELU2}


def _names(defaults: dict, given, what: str) -> dict:
    unknown = set(given or {}) - set(defaults)
    if unknown:
        raise ValueError(f"{what}: no tensor role named {sorted(unknown)}")
    out = dict(defaults)
    out.update(given or {})
    return out


class RoutedExperts(FeedForward):
    """params: hidden, experts, top_k, intermediate, score ("sigmoid" | "softmax"), correction_bias (bool: a bias on the pick
    keys only), logit_bias (bool: a bias that is part of the router's logits), normalize (bool), scale, names ({role: name
    below the prefix}), files ("fused" | "per_expert": how a model folder of the design holds the experts, for when no file says).  score "softmax" with normalize "always" is the softmax over the picked logits alone, for any top_k.
    unit ("swiglu", the default: silu(gate) * up | "clamped_glu": g = min(gate, limit), u = clamp(up, -limit, limit),
    g sigmoid(1.702 g) (u + 1)) with limit; weight_on ("output", the default: the row's result is sum_j w_j expert_j(h) |
    "input": sum_j expert_j(w_j h), the weight multiplying what the expert reads; the first product being linear, it is
    applied to both pre-activations before the unit); shared ({intermediate, limit (for clamped_glu), switch (bool)}: an
    expert of the same unit that every row runs, added to the routed sum, times sigmoid(W_switch h) (one number a row)
    where it has a switch).  unit "relu2": an expert is W_down max(W_up h, 0)^2, with no gate tensor (no shared expert
    or weight on the input is built for it); "geglu_tanh": the tanh form of gelu(gate) * up."""
    graph_safe = True

    wants_f32_input = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden = int(p["hidden"])
        self.experts = int(p["experts"])
        self.top_k = int(p["top_k"])
        self.intermediate = int(p["intermediate"])
        if p.get("score", "sigmoid") not in _SCORES:
            raise ValueError(f"router score {p.get('score')!r} is not one of {sorted(_SCORES)}")
        self.score = _SCORES[p.get("score", "sigmoid")]
        self.use_bias = bool(p.get("correction_bias", False))
        self.use_logit_bias = bool(p.get("logit_bias", False))
        self.names = _names(_EXPERT_NAMES, p.get("names"), "routed experts")
        self.files = str(p.get("files", "fused"))
        if self.files not in ("fused", "per_expert"):
            raise ValueError(f"routed experts: files {self.files!r} is not one of ['fused', 'per_expert']")
        given = p.get("normalize", True)
        self.normalize = "always" if given == "always" else bool(given)      # "always": one softmax pick is divided by itself too
        self.scale = float(p.get("scale", 1.0))
        if not 0 < self.top_k <= self.experts:
            raise ValueError("experts per token must be between 1 and the expert count")
        if self.experts > MAX_EXPERTS or self.top_k > MAX_TOP_K:
            raise ValueError(f"routed experts: {self.experts} experts with {self.top_k} picks a token; the routing kernels take at most "
                             f"{MAX_EXPERTS} experts and {MAX_TOP_K} picks")
        if p.get("unit", "swiglu") not in _UNITS and p.get("unit") not in _PLAIN_UNITS:
            raise ValueError(f"routed experts: unit {p.get('unit')!r} is not one of {sorted(list(_UNITS) + list(_PLAIN_UNITS))}")
        self.plain_unit = _PLAIN_UNITS.get(p.get("unit"))         # None: a gated unit
        self.unit = _UNITS.get(p.get("unit", "swiglu"), ops.GLU_SILU)
        self.limit = float(p.get("limit") or 0.0)
        if self.unit == ops.GLU_CLAMPED and not self.limit > 0.0:
            raise ValueError("routed experts: the clamped unit needs a positive limit")
        self.weight_on = str(p.get("weight_on", "output"))
        if self.weight_on not in ("output", "input"):
            raise ValueError(f"routed experts: weight_on {self.weight_on!r} is not one of ['input', 'output']")
        shared = p.get("shared")
        self.shared_width = int(shared["intermediate"]) if shared else 0
        self.shared_limit = float(shared.get("limit") or 0.0) if shared else 0.0
        self.shared_switch = bool(shared.get("switch", False)) if shared else False
        if self.plain_unit is not None and (shared or self.weight_on == "input"):
            raise ValueError("routed experts: a unit without a gate goes without a shared expert and with the weight on the output")
        if shared and (self.shared_width < 1 or (self.unit == ops.GLU_CLAMPED and not self.shared_limit > 0.0)):
            raise ValueError("routed experts: a shared expert has an inner width of at least 1 and, for the clamped unit, a positive limit")
        self.per_expert = False
        self.w_router = self.bias = self.logit_bias = self.w_gate_up = self.w_down = None
        self.w_shared_gate_up = self.w_shared_down = self.w_switch = None

    def tensor_specs(self, available):
        X, F, E = self.experts, self.intermediate, self.hidden
        nm = lambda role, **kw: self.name(self.names[role].format(**kw))
        specs = [TensorSpec(nm("router"), (X, E), "router")]
        if self.use_bias:
            specs.append(TensorSpec(nm("correction_bias"), (X,), "bias"))
        if self.use_logit_bias:
            specs.append(TensorSpec(nm("logit_bias"), (X,), "bias"))
        fused = nm("fused_gate_up")
        if self.plain_unit is not None:        # one product before the activation: the fused tensor holds the up rows alone
            head, _, tail = self.names["expert_up"].partition("{e}")
            single = re.compile(re.escape(self.name(head)) + r"\d+" + re.escape(tail) + "$")
            has_single = any(single.match(n) for n in available)
            self.per_expert = has_single or (self.files == "per_expert" and fused not in available)
            down = nm("fused_down")
            if self.per_expert:
                for e in range(X):
                    specs += [TensorSpec(nm("expert_up", e=e), (F, E), into=(fused, (X, F, E), (e,))),
                              TensorSpec(nm("expert_down", e=e), (E, F), into=(down, (X, E, F), (e,)))]
            else:
                specs += [TensorSpec(fused, (X, F, E)), TensorSpec(down, (X, E, F))]
            return specs
        head, _, tail = self.names["expert_gate"].partition("{e}")
        single = re.compile(re.escape(self.name(head)) + r"\d+" + re.escape(tail) + "$")
        has_single = any(single.match(n) for n in available)
        if has_single and fused in available:
            raise ValueError(f"{self.prefix}experts holds both fused and per-expert tensors")
        # a design whose files hold a tensor an expert is listed so also where no file is at hand (random weights)
        self.per_expert = has_single or (self.files == "per_expert" and fused not in available)
        if self.per_expert:
            # each expert's tensors go from the host straight into their places in the fused tensors
            down = nm("fused_down")
            for e in range(X):
                specs += [TensorSpec(nm("expert_gate", e=e), (F, E), into=(fused, (X, 2 * F, E), (e, slice(0, F)))),
                          TensorSpec(nm("expert_up", e=e), (F, E), into=(fused, (X, 2 * F, E), (e, slice(F, 2 * F)))),
                          TensorSpec(nm("expert_down", e=e), (E, F), into=(down, (X, E, F), (e,)))]
        else:
            specs += [TensorSpec(fused, (X, 2 * F, E)), TensorSpec(nm("fused_down"), (X, E, F))]
        if self.shared_width:
            S = self.shared_width
            shared = self.name("shared_gate_up")     # gate rows, then up rows, filled from the file's two tensors
            specs += [TensorSpec(nm("shared_gate"), (S, E), into=(shared, (2 * S, E), (slice(0, S),))),
                      TensorSpec(nm("shared_up"), (S, E), into=(shared, (2 * S, E), (slice(S, 2 * S),))),
                      TensorSpec(nm("shared_down"), (E, S))]
            if self.shared_switch:
                specs.append(TensorSpec(nm("shared_switch"), (1, E), "router"))
        return specs

    def load(self, tensors):
        self.w_router = tensors[self.name(self.names["router"])]
        if self.use_bias:
            self.bias = tensors[self.name(self.names["correction_bias"])]
        if self.use_logit_bias:
            self.logit_bias = tensors[self.name(self.names["logit_bias"])]
        # per-expert files arrive fused too (see tensor_specs)
        self.w_gate_up = tensors[self.name(self.names["fused_gate_up"])]
        self.w_down = tensors[self.name(self.names["fused_down"])]
        if self.shared_width:
            self.w_shared_gate_up = tensors[self.name("shared_gate_up")]
            self.w_shared_down = tensors[self.name(self.names["shared_down"])]
            if self.shared_switch:
                self.w_switch = tensors[self.name(self.names["shared_switch"])]

    def takes_deferred_norm(self, step):
        if self.shared_width or self.unit != ops.GLU_SILU or self.weight_on == "input" or self.plain_unit is not None:
            return False           # the shared expert's products and the other gated units read the rows as tensors
        return (ops.gemm_takes_normed_rows(step.rows, self.w_gate_up, step.act_dtype, ops.EPI_SWIGLU, grouped=True)
                and ops.gemm_f32_takes_normed_rows(step.rows, self.w_router))

    def forward(self, step, h, out, accumulate, h32=None):
        T, X, k = step.rows, self.experts, self.top_k
        z = step.buf("experts.router_logits", (T, X), torch.float32)
        slices = ops.gemm_f32_slices(X, h32.shape[1])
        parts = step.buf("experts.router_parts", (slices, T, X), torch.float32) if slices > 1 else None
        ops.gemm_f32(h32, self.w_router, z, parts=parts)
        ids = step.buf("experts.ids", (T, k), torch.int32)
        weights = step.buf("experts.weights", (T, k), torch.float32)
        counts = step.buf("experts.counts", (X,), torch.int32)
        offsets = step.buf("experts.offsets", (X + 1,), torch.int32)
        pairs = step.buf("experts.pairs", (T * k,), torch.int32)
        active = step.buf("experts.active", (X,), torch.int32)
        n_active = step.buf("experts.n_active", (1,), torch.int32)
        need = ops.moe_align_scratch(T * k, X)
        scratch = step.buf("experts.align_scratch", (need,), torch.int32) if need else None
        # for steps of many pairs the grouping also counts the experts' tiles of 128 rows, by which the products choose their tiles
        tile_stats = step.buf("experts.tile_stats", (1,), torch.int32) if T * k >= ops.TILE_STATS_MIN_PAIRS else None
        ops.route_topk_align(z, self.bias, ids, weights, k, self.score, self.normalize, self.scale, counts, offsets, pairs, active, n_active,
                             parts=parts, scratch=scratch, tile_stats=tile_stats, logit_bias=self.logit_bias)
        step.observe("routing", logits=z, ids=ids, weights=weights)
        act = step.buf("experts.act", (T * k, self.intermediate), step.act_dtype)
        on_input = self.weight_on == "input"
        if self.plain_unit is not None:
            ops.grouped_gemm(h, self.w_gate_up, act, offsets, pairs, k, ops.EPI_STORE, active, n_active, token_rows=T, tile_stats=tile_stats,
                             act=(self.plain_unit, None))
        else:
            glu = ops.Glu(self.unit, self.limit, weights.view(T * k) if on_input else None)
            ops.grouped_gemm(h, self.w_gate_up, act, offsets, pairs, k, ops.EPI_SWIGLU, active, n_active, token_rows=T, tile_stats=tile_stats,
                             glu=glu, scratch=step.buf)
        y = step.buf("experts.y", (T * k, self.hidden), torch.float32)
        ops.grouped_gemm(act, self.w_down, y, offsets, pairs, 1, ops.EPI_STORE, active, n_active, token_rows=T, tile_stats=tile_stats)
        ops.moe_combine(out, y, ids, None if on_input else weights, accumulate)
        if self.shared_width:
            # the shared expert: its switch is a factor on the rows its second product reads (that product is linear), so the
            # product can add straight into the routed sum
            switch = None
            if self.w_switch is not None:
                switch = step.buf("experts.switch", (T, 1), torch.float32)
                ops.gemm_f32(h32, self.w_switch, switch)
            shared = step.buf("experts.shared_act", (T, self.shared_width), step.act_dtype)
            ops.gemm(h, self.w_shared_gate_up, shared, ops.EPI_SWIGLU, glu=ops.Glu(self.unit, self.shared_limit, None, switch), scratch=step.buf)
            ops.gemm(shared, self.w_shared_down, out, ops.EPI_ADD, scratch=step.buf)


class DenseGLU(FeedForward):
    """params: hidden, intermediate, names ({role: name below the prefix}), unit ("swiglu", the default | "geglu_tanh": the
    tanh form of gelu on the gate).  y = (silu(h.Wg^T) * (h.Wu^T)).Wd^T; tensors gate_proj, up_proj, down_proj (.weight)
    unless named otherwise."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        self.names = _names(_GLU_NAMES, params.get("names"), "dense GLU")
        if params.get("unit", "swiglu") not in ("swiglu", "geglu_tanh"):
            raise ValueError(f"dense GLU: unit {params.get('unit')!r} is not one of ['geglu_tanh', 'swiglu']")
        self.glu = ops.Glu(_UNITS[params["unit"]]) if params.get("unit", "swiglu") != "swiglu" else None
        self.w_gate_up = self.w_down = None

    def tensor_specs(self, available):
        F, E = self.intermediate, self.hidden
        fused = self.name("gate_up_proj.weight")     # gate rows, then up rows, filled from the file's two tensors
        return [TensorSpec(self.name(self.names["gate"]), (F, E), into=(fused, (2 * F, E), (slice(0, F),))),
                TensorSpec(self.name(self.names["up"]), (F, E), into=(fused, (2 * F, E), (slice(F, 2 * F),))),
                TensorSpec(self.name(self.names["down"]), (E, F))]

    def load(self, tensors):
        self.w_gate_up = tensors[self.name("gate_up_proj.weight")]
        self.w_down = tensors[self.name(self.names["down"])]

    def takes_deferred_norm(self, step):
        return self.glu is None and ops.gemm_takes_normed_rows(step.rows, self.w_gate_up, step.act_dtype, ops.EPI_SWIGLU)

    def forward(self, step, h, out, accumulate, h32=None):
        act = step.buf("glu.act", (step.rows, self.intermediate), step.act_dtype)
        ops.gemm(h, self.w_gate_up, act, ops.EPI_SWIGLU, glu=self.glu)
        ops.gemm(act, self.w_down, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


class DenseAct(FeedForward):
    """params: hidden, intermediate, activation ("xielu" | "polynorm"), eps (polynorm).  y = W_down act(W_up h); tensors
    <prefix>up, down, and <prefix>act: for xIELU (p, q): act(z) = softplus(p) z^2 + z/2 for z > 0, (1/2 + softplus(q))
    (e^z - 1 - z) + z/2 otherwise; for polynorm (a, b, c, e): act(z) = a U(z) + b U(z^2) + c U(z^3) + e with powers element by
    element and U dividing a row of inner values by its root mean square (eps inside the root): it needs the whole row, so
    it is a kernel of its own between the two products, in float32."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        self.activation = str(params.get("activation", "xielu"))
        if self.activation not in ("xielu", "polynorm"):
            raise ValueError(f"dense feed-forward: activation {self.activation!r} is not one of ['polynorm', 'xielu']")
        self.eps = float(params.get("eps", 0.0))
        self.w_up = self.w_down = self.act = None

    def tensor_specs(self, available):
        F, E = self.intermediate, self.hidden
        numbers = 2 if self.activation == "xielu" else 4
        return [TensorSpec(self.name("up"), (F, E)), TensorSpec(self.name("down"), (E, F)),
                TensorSpec(self.name("act"), (numbers,), "bias", dtype="float32", init=("uniform", -1.0, 1.0))]

    def load(self, tensors):
        self.w_up = tensors[self.name("up")]
        self.w_down = tensors[self.name("down")]
        self.act = tensors[self.name("act")]

    def forward(self, step, h, out, accumulate, h32=None):
        a = step.buf("dense.act", (step.rows, self.intermediate), step.act_dtype)
        if self.activation == "polynorm":
            z = step.buf("dense.pre", (step.rows, self.intermediate), torch.float32)
            ops.gemm(h, self.w_up, z, scratch=step.buf)
            ops.act_polynorm(z, self.act, self.eps, a)
        else:
            ops.gemm(h, self.w_up, a, scratch=step.buf, act=(ops.ACT_XIELU, self.act))      # the activation in the product's epilogue
        ops.gemm(a, self.w_down, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("feed_forward", "routed_experts", RoutedExperts)
register("feed_forward", "dense_act", DenseAct)
register("feed_forward", "dense_glu", DenseGLU)
