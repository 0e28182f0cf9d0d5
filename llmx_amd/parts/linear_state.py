"""Mixers that carry a float32 matrix state S [key channels D, value channels V] a head from token to token.

All decay S's rows (channel by channel, or a head's all alike) and add an outer product a token; they differ in what is added:
    S_t = diag(g_t) S_(t-1) + k_t u_t^T,   o_t = S_t^T q_t
    gated linear attention:  u_t = v_t,                               g_t = sigmoid(z_t)^(1/tau)
    gated delta rule:        u_t = beta_t (v_t - (diag(g_t) S_(t-1))^T k_t),   g_t = exp(-exp(A) softplus(step_t + dt_bias))
with z_t and step_t low-rank projections of the input.  The delta rule's q, k and v first pass a short causal convolution
over time and silu, and q and k are made unit vectors a head.  The read-out is RMS-normed a head, gated, and projected.
Products may read rounded rows; decays, gates, unit norms, the recurrence and the state are float32 in both paths.
The state lives in the request's slot: S (in the scan kernel's tiles of value channels), then (delta rule) the convolution's
last taps - 1 inputs [taps - 1, C].
"""

from __future__ import annotations

import torch

from .. import ops
from .base import LayerCache, Mixer, register
from .spec import StateNeed, TensorSpec


class GatedLinearAttention(Mixer):
    """params: hidden, heads, dim, vdim, tau, eps, rank (the decay projection's inner width).
    q = W_q h * dim^-1/2, k = W_k h, v = W_v h; decay = sigmoid(W_a2 (W_a1 h) + b)^(1/tau) a key channel;
    result = W_o (rmsnorm_head(o) * w * silu(W_g h)).  Tensors <prefix>q, k, v, g, o, norm, a1, a2, a2.b."""
    graph_safe = True
    steps_between_slots = True      # reads the state at step.entry_held_slots, writes it at step.entry_slots

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden, self.heads, self.dim, self.vdim = int(p["hidden"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.rank = int(p["rank"])
        self.tau, self.eps = float(p["tau"]), float(p["eps"])
        if min(self.heads, self.dim, self.vdim, self.rank) < 1 or self.dim > 256 or not self.tau > 0.0:
            raise ValueError("gated linear attention: heads, dim (at most 256), vdim and rank are at least 1 and tau is positive")
        HD, HV = self.heads * self.dim, self.heads * self.vdim
        # the fused in-projection's columns: q | k | v | g | a1
        self.cols = {"q": (0, HD), "k": (HD, HD), "v": (2 * HD, HV), "g": (2 * HD + HV, HV), "a1": (2 * HD + 2 * HV, self.rank)}
        self.in_width = 2 * HD + 2 * HV + self.rank
        self.w_in = self.w_a2 = self.b_a2 = self.w_o = self.norm = None

    def cache_need(self):
        return StateNeed((ops.state_matrix_size(self.heads, self.dim, self.vdim),), "float32")

    def tensor_specs(self, available):
        E = self.hidden
        fused, shape = self.name("in"), (self.in_width, E)
        specs = [TensorSpec(self.name(n), (w, E), into=(fused, shape, (slice(at, at + w),))) for n, (at, w) in self.cols.items()]
        return specs + [TensorSpec(self.name("a2"), (self.heads * self.dim, self.rank)),
                        TensorSpec(self.name("a2.b"), (self.heads * self.dim,), "bias"),
                        TensorSpec(self.name("norm"), (self.vdim,), "norm"),
                        TensorSpec(self.name("o"), (E, self.heads * self.vdim))]

    def load(self, tensors):
        self.w_in = tensors[self.name("in")]
        self.w_a2, self.b_a2 = tensors[self.name("a2")], tensors[self.name("a2.b")]
        self.norm, self.w_o = tensors[self.name("norm")], tensors[self.name("o")]

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T, H, D, V = step.rows, self.heads, self.dim, self.vdim
        pre = step.buf("gla.pre", (T, self.in_width), torch.float32)
        ops.gemm(h, self.w_in, pre, scratch=step.buf)
        view = lambda n: pre[:, self.cols[n][0]:self.cols[n][0] + self.cols[n][1]]
        # the low-rank projection's inner values as rows of their own, in the type products read
        inner = step.buf("gla.inner", (T, self.rank), step.act_dtype)
        ops.cast_cols(view("a1"), inner)
        z = step.buf("gla.z", (T, H * D), torch.float32)
        ops.gemm(inner, self.w_a2, z, scratch=step.buf)
        decay = step.buf("gla.decay", (T, H * D), torch.float32)
        ops.sigmoid_root(z, self.b_a2, self.tau, decay)
        o = step.buf("gla.o", (T, H * V), torch.float32)
        ops.state_scan(view("q"), view("k"), view("v"), decay, None, cache.state, step.entry_held_slots, step.entry_slots, step.entry_rows, o,
                       float(D) ** -0.5, H, H, D, V, max_rows=step.max_rows_per_entry)
        gated = step.buf("gla.gated", (T, H * V), step.act_dtype)
        ops.head_norm_gate(o, self.norm, view("g"), gated, self.eps, H, V, ops.GATE_SILU)
        ops.gemm(gated, self.w_o, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


class ChannelDeltaRule(Mixer):
    """params: hidden, heads, kv_heads (q and k heads; head h reads q/k head h / (heads / kv_heads)), dim, vdim, conv (taps),
    eps, decay_rank, gate_rank.  Tensors <prefix>q, k, v (+ .conv [channels, taps]), b, A_log, dt_bias, a1, a2, g1, g2,
    norm, o.  result = W_o (rmsnorm_head(o) * w * sigmoid(W_g2 (W_g1 h)))."""
    graph_safe = True
    steps_between_slots = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden, self.heads, self.kv_heads = int(p["hidden"]), int(p["heads"]), int(p["kv_heads"])
        self.dim, self.vdim, self.taps = int(p["dim"]), int(p["vdim"]), int(p["conv"])
        self.decay_rank, self.gate_rank = int(p["decay_rank"]), int(p["gate_rank"])
        self.eps = float(p["eps"])
        if min(self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.decay_rank, self.gate_rank) < 1 or self.dim > 256:
            raise ValueError("delta rule: heads, kv_heads, dim (at most 256), vdim, conv and the ranks are at least 1")
        if self.heads % self.kv_heads:
            raise ValueError("delta rule: the head count must be divisible by the q/k head count")
        GD, HV, H = self.kv_heads * self.dim, self.heads * self.vdim, self.heads
        self.channels = 2 * GD + HV
        # the fused in-projection's columns: q | k | v (the convolved channels, in this order) | b | a1 | g1
        self.cols = {"q": (0, GD), "k": (GD, GD), "v": (2 * GD, HV), "b": (self.channels, H), "a1": (self.channels + H, self.decay_rank),
                     "g1": (self.channels + H + self.decay_rank, self.gate_rank)}
        self.in_width = self.channels + H + self.decay_rank + self.gate_rank
        self.state_matrix = ops.state_matrix_size(H, self.dim, self.vdim)
        self.w_in = self.conv = self.a_log = self.dt_bias = self.w_low = self.norm = self.w_o = None

    def cache_need(self):
        return StateNeed((self.state_matrix + (self.taps - 1) * self.channels,), "float32")

    def tensor_specs(self, available):
        E, H, D, V = self.hidden, self.heads, self.dim, self.vdim
        fused, shape = self.name("in"), (self.in_width, E)
        specs = [TensorSpec(self.name(n), (w, E), into=(fused, shape, (slice(at, at + w),))) for n, (at, w) in self.cols.items()]
        taps_of, taps_shape = self.name("conv"), (self.channels, self.taps)
        specs += [TensorSpec(self.name(f"{n}.conv"), (self.cols[n][1], self.taps), "bias",
                             into=(taps_of, taps_shape, (slice(self.cols[n][0], self.cols[n][0] + self.cols[n][1]),)), init=("uniform", -0.5, 0.5))
                  for n in ("q", "k", "v")]
        return specs + [TensorSpec(self.name("A_log"), (H,), "bias", init=("uniform", -1.0, 1.0)),
                        TensorSpec(self.name("dt_bias"), (H * D,), "bias"),
                        TensorSpec(self.name("a2"), (H * D, self.decay_rank)),
                        TensorSpec(self.name("g2"), (H * V, self.gate_rank)),
                        TensorSpec(self.name("norm"), (V,), "norm"),
                        TensorSpec(self.name("o"), (E, H * V))]

    def load(self, tensors):
        self.w_in, self.conv = tensors[self.name("in")], tensors[self.name("conv")]
        self.a_log, self.dt_bias = tensors[self.name("A_log")], tensors[self.name("dt_bias")]
        # the two low-rank projections' second halves as one product: [step | gate] = [a1 h | g1 h] @ blockdiag(a2, g2)^T
        a2, g2 = tensors[self.name("a2")], tensors[self.name("g2")]
        self.w_low = torch.zeros((a2.shape[0] + g2.shape[0], self.decay_rank + self.gate_rank), dtype=a2.dtype, device=a2.device)
        self.w_low[:a2.shape[0], :self.decay_rank].copy_(a2)
        self.w_low[a2.shape[0]:, self.decay_rank:].copy_(g2)
        self.norm, self.w_o = tensors[self.name("norm")], tensors[self.name("o")]

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T, H, G, D, V = step.rows, self.heads, self.kv_heads, self.dim, self.vdim
        f32 = torch.float32
        pre = step.buf("delta.pre", (T, self.in_width), f32)
        ops.gemm(h, self.w_in, pre, scratch=step.buf)
        view = lambda n: pre[:, self.cols[n][0]:self.cols[n][0] + self.cols[n][1]]
        # both low-rank projections' inner values (neighbouring columns) as rows of their own, in the type products read
        ranks = self.decay_rank + self.gate_rank
        inner = step.buf("delta.inner", (T, ranks), step.act_dtype)
        ops.cast_cols(pre[:, self.cols["a1"][0]:self.cols["a1"][0] + ranks], inner)
        low = step.buf("delta.low", (T, H * D + H * V), f32)
        ops.gemm(inner, self.w_low, low, scratch=step.buf)
        step_pre, gate_pre = low[:, :H * D], low[:, H * D:]
        q, k = step.buf("delta.q", (T, G * D), f32), step.buf("delta.k", (T, G * D), f32)
        v, decay, beta = step.buf("delta.v", (T, H * V), f32), step.buf("delta.decay", (T, H * D), f32), step.buf("delta.beta", (T, H), f32)
        ops.delta_prep(pre, self.conv, step_pre, self.dt_bias, self.a_log, cache.state, self.state_matrix, step.entry_held_slots,
                       step.row_entry, step.entry_rows, q, k, v, decay, beta, G, H, D, V, self.cols["b"][0])
        o = step.buf("delta.o", (T, H * V), f32)
        tail = (pre[:, :self.channels], self.taps, self.state_matrix) if self.taps > 1 else None
        ops.state_scan(q, k, v, decay, beta, cache.state, step.entry_held_slots, step.entry_slots, step.entry_rows, o, float(D) ** -0.5,
                       H, G, D, V, tail=tail, max_rows=step.max_rows_per_entry)
        gated = step.buf("delta.gated", (T, H * V), step.act_dtype)
        ops.head_norm_gate(o, self.norm, gate_pre, gated, self.eps, H, V, ops.GATE_SIGMOID)
        ops.gemm(gated, self.w_o, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


class GatedMatrixMemory(Mixer):
    """A matrix memory a head with an exponential input gate and a sigmoid forget gate, kept in range by a running maximum m
    (which starts at 0):
        i_t = cap tanh((W_i h + b_i) / cap),   f_t = log sigmoid(cap tanh((W_f h + b_f) / cap)),   m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),   q_t = W_q h dim^-1/2
    result = W_o (o / rms(o) a head * w * sigmoid(W_g h)), w of all heads' width.  params: hidden, heads, dim, vdim, gate_cap,
    eps.  Tensors <prefix>q, k, v, g, i, f, i.b, f.b, norm, o.  This is the scan's recurrence with one decay for all of a
    head's key channels, keys times exp(i_t - m_t) and one more value channel that is always 1, whose column of S is n; the
    state slot holds that S (in the scan's tiles), then m, one float a head.  Gates, exponentials, the recurrence, its
    state and the read-out's norm are float32 in both paths."""
    graph_safe = True
    steps_between_slots = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden, self.heads, self.dim, self.vdim = int(p["hidden"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        if min(self.heads, self.dim, self.vdim) < 1 or self.dim > 256 or not self.cap > 0.0:
            raise ValueError("gated matrix memory: heads, dim (at most 256) and vdim are at least 1 and gate_cap is positive")
        H, HD, HV = self.heads, self.heads * self.dim, self.heads * self.vdim
        # the fused in-projection's columns: q | k | v | g | i | f
        self.cols = {"q": (0, HD), "k": (HD, HD), "v": (2 * HD, HV), "g": (2 * HD + HV, HV), "i": (2 * HD + 2 * HV, H), "f": (2 * HD + 2 * HV + H, H)}
        self.in_width = 2 * HD + 2 * HV + 2 * H
        self.state_matrix = ops.state_matrix_size(H, self.dim, self.vdim + 1)
        self.w_in = self.b_i = self.b_f = self.norm = self.w_o = None

    def cache_need(self):
        return StateNeed((self.state_matrix + self.heads,), "float32")

    def tensor_specs(self, available):
        E = self.hidden
        fused, shape = self.name("in"), (self.in_width, E)
        specs = [TensorSpec(self.name(n), (w, E), into=(fused, shape, (slice(at, at + w),))) for n, (at, w) in self.cols.items()]
        return specs + [TensorSpec(self.name("i.b"), (self.heads,), "bias"), TensorSpec(self.name("f.b"), (self.heads,), "bias"),
                        TensorSpec(self.name("norm"), (self.heads * self.vdim,), "norm"),
                        TensorSpec(self.name("o"), (E, self.heads * self.vdim))]

    def load(self, tensors):
        self.w_in = tensors[self.name("in")]
        self.b_i, self.b_f = tensors[self.name("i.b")], tensors[self.name("f.b")]
        self.norm, self.w_o = tensors[self.name("norm")], tensors[self.name("o")]

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T, H, D, V = step.rows, self.heads, self.dim, self.vdim
        f32 = torch.float32
        pre = step.buf("memory.pre", (T, self.in_width), f32)
        ops.gemm(h, self.w_in, pre, scratch=step.buf)
        view = lambda n: pre[:, self.cols[n][0]:self.cols[n][0] + self.cols[n][1]]
        decay, keys = step.buf("memory.decay", (T, H * D), f32), step.buf("memory.keys", (T, H * D), f32)
        values, floor = step.buf("memory.values", (T, H * (V + 1)), f32), step.buf("memory.floor", (T, H), f32)
        ops.memory_prep(pre, {n: at for n, (at, _) in self.cols.items()}, self.b_i, self.b_f, self.cap, cache.state, self.state_matrix,
                        step.entry_held_slots, step.entry_slots, step.entry_rows, decay, keys, values, floor, H, D, V,
                        factors=step.buf("memory.factors", (T, H, 2), f32))
        o = step.buf("memory.o", (T, H * (V + 1)), f32)
        ops.state_scan(view("q"), keys, values, decay, None, cache.state, step.entry_held_slots, step.entry_slots, step.entry_rows, o,
                       float(D) ** -0.5, H, H, D, V + 1, max_rows=step.max_rows_per_entry)
        gated = step.buf("memory.gated", (T, H * V), step.act_dtype)
        ops.head_norm_gate(o, self.norm, view("g"), gated, self.eps, H, V, ops.GATE_SIGMOID, den_floor=floor)
        ops.gemm(gated, self.w_o, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "gated_matrix_memory", GatedMatrixMemory)
register("mixer", "gated_linear_attention", GatedLinearAttention)
register("mixer", "channel_delta_rule", ChannelDeltaRule)
