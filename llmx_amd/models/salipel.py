"""Salipel assembled from parts.

Embedding; per layer the "parallel" arrangement with one RMS norm whose rows both sublayers read and a constant on their
sum (x += m (mixer(h) + ff(h)), h = norm1(x)); a mixer among attention in chunks (distance slopes, a sink, unit-RMS
values, no rotation), attention with two score maps a head (soft-capped, the difference normed and gated), and a windowed
attention that keeps the first tokens (values = the projected keys, a gate a value) side by side with a gated matrix
memory; a dense gated unit with the tanh form of gelu, routed squared-relu experts (softmax scores, a correction on the
choice, weights normalized and scaled) or no feed-forward; a final RMS norm and an untied head.
Tensor names: embed, l<i>.norm1, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""

from __future__ import annotations

from ..config.salipel import ARCHITECTURE, SalipelConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry
from .registry import register_architecture

NO_POSITION_LIMIT = 1 << 30     # the design states no longest context: the cache's size is the limit

_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "output_gate": "g", "sink": "sink",
                    "lambda_q1": "lq1", "lambda_k1": "lk1", "lambda_q2": "lq2", "lambda_k2": "lk2"}
_EXPERT_NAMES = {"router": "router", "correction_bias": "correction", "expert_up": "e{e}.up", "expert_down": "e{e}.down",
                 "fused_gate_up": "up", "fused_down": "down"}
_GLU_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _rotation(rot) -> PartSpec:
    s = rot.scaling
    return PartSpec("rotary_scaled", {"dims": rot.dims, "base": rot.base, "pairing": "halves",
                                      "scaling": None if s is None else {"factor": s.factor, "low": s.low, "high": s.high,
                                                                         "original": s.original}})


def _mixer(c: SalipelConfig, i: int) -> PartSpec:
    layer = c.layers[i]
    m, p = layer.mixer, f"l{i}.mix."
    common = {"hidden": c.width, "eps": c.norm_eps, "names": _ATTENTION_NAMES}
    if layer.type == "attention":
        return PartSpec("attention", dict(common, heads=m.heads, kv_heads=m.kv_heads, head_dim=m.dim, v_dim=m.vdim, scale=m.scale,
                                          qk_norm="none", chunk=m.chunk, distance_slopes=True, sink=True, value_norm=True), p)
    if layer.type == "attention_2":
        return PartSpec("attention", dict(common, heads=m.heads, kv_heads=m.kv_heads, head_dim=m.dim, v_dim=m.vdim, scale=m.scale,
                                          qk_norm="head", softcap=m.softcap, difference={"diff": m.diff}, output_gate=True,
                                          position=_rotation(m.rot)), p)
    a, b = m.left, m.right
    left = PartSpec("attention", dict(common, heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, v_dim=a.vdim, scale=a.scale,
                                      qk_norm="head", window=a.window, keep_first=a.keep_first, values="keys", output_gate=True,
                                      position=_rotation(a.rot)), p + "left.")
    right = PartSpec("gated_matrix_memory", {"hidden": c.width, "heads": b.heads, "dim": b.dim, "vdim": b.vdim, "gate_cap": b.gate_cap,
                                             "eps": c.norm_eps}, p + "right.")
    return PartSpec("side_by_side", {"hidden": c.width, "members": [{"name": "left", "scale": m.left_scale, "mixer": left},
                                                                    {"name": "right", "scale": m.right_scale, "mixer": right}]}, p)


def assemble(c: SalipelConfig) -> ModelSpec:
    E = c.width

    def norm(name):
        return PartSpec("rmsnorm", {"width": E, "eps": c.norm_eps, "tensor": ""}, name)

    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        ffn = None
        if layer.mlp is not None:
            if layer.mlp.kind == "dense":
                ffn = PartSpec("dense_glu", {"hidden": E, "intermediate": layer.mlp.ff, "unit": "geglu_tanh", "names": _GLU_NAMES}, p + "mlp.")
            else:
                ffn = PartSpec("routed_experts", {"hidden": E, "experts": layer.mlp.experts, "top_k": layer.mlp.top, "intermediate": layer.mlp.ff,
                                                  "score": "softmax", "correction_bias": True, "normalize": "always", "scale": layer.mlp.scale,
                                                  "unit": "relu2", "names": _EXPERT_NAMES, "files": "per_expert"}, p + "mlp.")
        # one norm: the feed-forward has none of its own and reads the mixer's normed rows
        scale = ("scale", PartSpec("constant", {"value": c.residual_mult}))
        blocks.append(BlockSpec(mixer_norm=norm(p + "norm1"), mixer=_mixer(c, i), ffn_norm=None, ffn=ffn, arrangement="parallel",
                                extra={"mixer_scale": scale, "ffn_scale": scale} if ffn is not None else {"mixer_scale": scale}))
    return ModelSpec(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=E,
        max_positions=NO_POSITION_LIMIT,
        embedding=PartSpec("token_embedding", {"vocab": c.vocab, "hidden": E, "tensor": ""}, "embed"),
        blocks=blocks,
        run_order=[RunEntry(layer=i, cache=i) for i in range(len(blocks))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab": c.vocab, "hidden": E, "tied": False, "tensor": ""}, "head"),
    )


register_architecture(ARCHITECTURE, SalipelConfig, assemble, replace=True)
