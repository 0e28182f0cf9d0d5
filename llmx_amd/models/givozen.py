"""Givozen assembled from parts.

Embedding; per layer the "sandwich" arrangement (x += N1b(mixer(N1(x))); x += N2b(ff(N2(x))), N an RMS norm whose stored
weight lies around zero) with causal grouped-query attention (biased q, k, v; a partial rotation in halves with
frequencies rescaled by wavelength; a temperature and a sigmoid gate a head; values of their own width) and a feed-forward
among dense with a polynomial of unit-RMS powers, routed experts of a clamped gated unit whose sigmoid scores multiply
the expert's input (plus a shared expert behind a sigmoid switch), or none; a final norm and the embedding table as head.
A repeated run of layers becomes further run-order entries of the same blocks, each with a cache number of its own; the
first entry of a pass names the residual input that adds the pass's vector (and, from the second pass on, the embedding
rows).  Tensor names: embed, loop.step, l<i>.norm1|norm1b|norm2|norm2b, l<i>.mix.*, l<i>.mlp.*, final.norm.
"""

from __future__ import annotations

from ..config.givozen import ARCHITECTURE, GivozenConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry
from .registry import register_architecture

NO_POSITION_LIMIT = 1 << 30     # the design states no longest context: the cache's size is the limit

_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "head_temperature": "temp",
                    "head_gate": "g"}
_EXPERT_NAMES = {"router": "router", "expert_gate": "e{e}.gate", "expert_up": "e{e}.up", "expert_down": "e{e}.down",
                 "fused_gate_up": "gate_up", "fused_down": "down", "shared_gate": "shared.gate", "shared_up": "shared.up",
                 "shared_down": "shared.down", "shared_switch": "shared.sg"}


def _mixer(c: GivozenConfig, i: int) -> PartSpec:
    a = c.layers[i].mixer
    s = a.rot_scaling
    position = PartSpec("rotary_scaled", {"dims": a.rot_dims, "base": a.rot_base, "pairing": "halves",
                                          "scaling": None if s is None else {"factor": s.factor, "low": s.low, "high": s.high,
                                                                             "original": s.original}})
    return PartSpec("attention", {"hidden": c.width, "heads": a.heads, "kv_heads": a.kv_heads, "head_dim": a.dim, "v_dim": a.vdim,
                                  "qk_norm": "none", "scale": a.scale, "bias": "qkv", "head_temperature": True, "head_gate": True,
                                  "position": position, "names": _ATTENTION_NAMES}, f"l{i}.mix.")


def _feed_forward(c: GivozenConfig, i: int) -> PartSpec:
    mlp, p = c.layers[i].mlp, f"l{i}.mlp."
    if mlp.kind == "dense":
        return PartSpec("dense_act", {"hidden": c.width, "intermediate": mlp.ff, "activation": "polynorm", "eps": c.norm_eps}, p)
    shared = None if mlp.shared is None else {"intermediate": mlp.shared.ff, "limit": mlp.shared.limit, "switch": True}
    return PartSpec("routed_experts", {"hidden": c.width, "experts": mlp.experts, "top_k": mlp.top, "intermediate": mlp.ff,
                                       "score": "sigmoid", "normalize": False, "unit": "clamped_glu", "limit": mlp.limit,
                                       "weight_on": "input", "shared": shared, "names": _EXPERT_NAMES, "files": "per_expert"}, p)


def assemble(c: GivozenConfig) -> ModelSpec:
    E = c.width

    def norm(name):
        return PartSpec("rmsnorm", {"width": E, "eps": c.norm_eps, "tensor": "", "offset": 1.0}, name)

    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        extra = {"mixer_post": ("norm", norm(p + "norm1b"))}
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn_norm, ffn = norm(p + "norm2"), _feed_forward(c, i)
            extra["ffn_post"] = ("norm", norm(p + "norm2b"))
        blocks.append(BlockSpec(mixer_norm=norm(p + "norm1"), mixer=_mixer(c, i), ffn_norm=ffn_norm, ffn=ffn, arrangement="sandwich",
                                extra=extra))
    inputs, run_order = [], []
    for number, (i, t, opens) in enumerate(c.passes()):
        before = None
        if opens:
            before = len(inputs)
            inputs.append(PartSpec("pass_vector", {"hidden": E, "passes": c.loop.times, "index": t, "add_embedding": t > 0}, "loop.step"))
        run_order.append(RunEntry(layer=i, cache=number, before=before))
    return ModelSpec(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=E,
        max_positions=NO_POSITION_LIMIT,
        embedding=PartSpec("token_embedding", {"vocab": c.vocab, "hidden": E, "tensor": ""}, "embed"),
        blocks=blocks,
        run_order=run_order,
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab": c.vocab, "hidden": E, "tied": True}, "head"),
        inputs=inputs,
    )


register_architecture(ARCHITECTURE, GivozenConfig, assemble, replace=True)
