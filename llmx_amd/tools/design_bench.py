"""Prefill and decode throughput of one design beside the closest other one at equal size, with random weights.

`python bench.py --design bonerax` does the same for a Bonerax (layers in turn: windowed attention beside a delta rule,
gated linear attention, the delta rule alone; routed SwiGLU experts) and a MiniMax-M3 with the same width, layers, heads,
head width and experts.

`python bench.py --design givozen` does the same for a Givozen (a dense layer with the polynomial activation, then layers of
routed clamped-unit experts with a shared expert, two of them run twice; attention with biases, a temperature and a gate
a head) and a MiniMax-M3 with as many layers as the Givozen has layer runs and the same width, heads, head width, experts,
picks and expert width.  A repeated layer's weights count each time they run.

`python bench.py --design salipel` does the same for a Salipel (layers in turn: two score maps a head with a dense gated
unit, the same with routed squared-relu experts, windowed attention that keeps the first tokens beside a gated matrix memory,
attention in chunks with routed experts) and a MiniMax-M3 of the same width, layers, heads, experts, picks and expert width.

`python bench.py --design nenotar` measures, at sizes that resemble a real model's layers, a Nenotar (latent attention
and minGRU layers in turn, each with a dense xIELU feed-forward and a per-layer token input) and a MiniMax-M3 of the
same width, layers, heads and vocabulary whose routed experts hold the same active weights a token: one 2,048-token
prompt from an empty cache, and decode steps of 1 and 8 requests at a context of 4,096 tokens.  Each record has tok/s,
ms, the bytes a decode step must read (every weight once and the live cache) with their share of 8 TB/s, and a prompt's
floating-point work with its share of the bf16 peak.  One JSON line.
"""

from __future__ import annotations

import json
import time

HBM_PEAK_GBS = 8000.0
BF16_PEAK = 2.5e15
PROMPT = 2048
CONTEXT = 4096

# name -> (width, layers, heads, ff, recurrent width, token-input dim, vocab); a head is 128 unrotated + 64 rotated dims
# over a latent of 512, values of 128
SIZES = {
    "w2048": (2048, 8, 16, 8192, 3072, 128, 32768),
    "w4096": (4096, 4, 32, 16384, 6144, 256, 32768),
    "w256": (256, 2, 2, 768, 384, 16, 1024),        # seconds: for trying the option out; not among the default sizes
}
DEFAULT_SIZES = ("w2048", "w4096")


def nenotar_config(width, layers, heads, ff, recurrent, side, vocab):
    from llmx_amd import NenotarConfig
    from llmx_amd.config.nenotar import LatentAttentionConfig, LayerConfig, MinGRUConfig, RotaryScaling
    latent = LatentAttentionConfig(heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=512, scale=192 ** -0.5, rot_base=10000.0, rot_dims=64,
                                   rot_scaling=RotaryScaling(40.0, 4096.0, 32.0, 1.0))
    kinds = [LayerConfig("latent_attention", latent, ff) if i % 2 == 0 else LayerConfig("mingru", MinGRUConfig(recurrent), ff) for i in range(layers)]
    return NenotarConfig(vocab=vocab, width=width, embedding_scale=1.0, norm_eps=1e-6, layers=tuple(kinds), token_side_dim=side)


def closest_config(width, layers, heads, ff, recurrent, side, vocab):
    """MiniMax-M3 of the same width, layers, heads and vocabulary: 8 experts of which 2 a token, holding together the
    active weights of the dense feed-forward (2 x width x ff = 2 x 3 x width x intermediate)."""
    from llmx_amd import MiniMaxM3Config
    inter = max(64, (ff // 3) // 64 * 64)
    return MiniMaxM3Config(vocab_size=vocab, hidden_size=width, num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=max(1, heads // 4),
                           head_dim=128, rotary_dim=64, rope_theta=1e6, rms_norm_eps=1e-6, num_local_experts=8, num_experts_per_tok=2,
                           intermediate_size=inter, routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False,
                           max_position_embeddings=2 * CONTEXT)


# name -> (width, layers, attention heads, kv heads, window, recurrent heads (of 128 x 128), experts, picks, expert ff, vocab)
BONERAX_SIZES = {
    "w2048": (2048, 6, 16, 4, 1024, 16, 8, 2, 2048, 32768),
    "w4096": (4096, 3, 32, 8, 1024, 32, 8, 2, 4096, 32768),
    "w256": (256, 3, 2, 1, 64, 2, 4, 2, 128, 1024),
}


def bonerax_config(width, layers, heads, kv_heads, window, rec_heads, experts, top, ff, vocab):
    from llmx_amd.config.bonerax import (BoneraxConfig, DeltaConfig, GLAConfig, LayerConfig, MLPConfig, ParallelConfig, RotaryScaling,
                                         WindowAttentionConfig)
    left = WindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5, window=window, rot_base=10000.0,
                                 rot_dims=64, rot_scaling=RotaryScaling(8.0, 4096.0, 32.0, 1.0))
    delta = DeltaConfig(heads=rec_heads, kv_heads=rec_heads, dim=128, vdim=128, conv=4)
    kinds = [("parallel", ParallelConfig(left, DeltaConfig(heads=max(1, rec_heads // 4), kv_heads=max(1, rec_heads // 4), dim=128, vdim=128, conv=4),
                                         0.8, 0.9)),
             ("gla", GLAConfig(heads=rec_heads, dim=64, vdim=128, tau=16.0)), ("channel_delta", delta)]
    mlp = MLPConfig("moe", ff, experts=experts, top=top)
    rank = max(16, width // 32)
    return BoneraxConfig(vocab=vocab, width=width, norm_eps=1e-5, logit_scale=1.0, logit_softcap=30.0,
                         layers=tuple(LayerConfig(*kinds[i % 3], mlp) for i in range(layers)),
                         ranks={i: {"decay": rank, "gate": rank} for i in range(layers)})


def bonerax_closest(width, layers, heads, kv_heads, window, rec_heads, experts, top, ff, vocab):
    """MiniMax-M3 of the same width, layers, heads, head width, experts, picks and expert width."""
    from llmx_amd import MiniMaxM3Config
    return MiniMaxM3Config(vocab_size=vocab, hidden_size=width, num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv_heads,
                           head_dim=128, rotary_dim=64, rope_theta=1e6, rms_norm_eps=1e-6, num_local_experts=experts, num_experts_per_tok=top,
                           intermediate_size=ff, routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False,
                           max_position_embeddings=2 * CONTEXT)


# name -> (width, layers, heads, kv heads, dense ff, experts, picks, expert ff, shared ff, loop (start, stop, times), vocab)
GIVOZEN_SIZES = {
    "w2048": (2048, 6, 16, 4, 8192, 8, 2, 2048, 2048, (1, 3, 2), 32768),
    "w4096": (4096, 3, 32, 8, 16384, 8, 2, 4096, 4096, (1, 2, 2), 32768),
    "w256": (256, 3, 2, 1, 768, 4, 2, 128, 64, (1, 2, 2), 1024),
}


def givozen_config(width, layers, heads, kv_heads, dense_ff, experts, top, ff, shared_ff, loop, vocab):
    from llmx_amd.config.givozen import AttentionConfig, GivozenConfig, LayerConfig, LoopConfig, MLPConfig, SharedExpertConfig, WavelengthScaling
    mixer = AttentionConfig(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5, rot_base=1e6, rot_dims=64,
                            rot_scaling=WavelengthScaling(8.0, 1.0, 4.0, 8192.0))
    moe = MLPConfig("moe", ff, limit=7.0, experts=experts, top=top, shared=SharedExpertConfig(shared_ff, 7.0))
    kinds = [LayerConfig("attention", mixer, MLPConfig("dense", dense_ff) if i == 0 else moe) for i in range(layers)]
    return GivozenConfig(vocab=vocab, width=width, norm_eps=1e-6, layers=tuple(kinds), loop=LoopConfig(*loop))


def givozen_closest(width, layers, heads, kv_heads, dense_ff, experts, top, ff, shared_ff, loop, vocab):
    """MiniMax-M3 with a layer for every layer run of the Givozen, the same width, heads, head width, experts, picks and
    expert width."""
    from llmx_amd import MiniMaxM3Config
    runs = layers + (loop[1] - loop[0]) * (loop[2] - 1)
    return MiniMaxM3Config(vocab_size=vocab, hidden_size=width, num_hidden_layers=runs, num_attention_heads=heads, num_key_value_heads=kv_heads,
                           head_dim=128, rotary_dim=64, rope_theta=1e6, rms_norm_eps=1e-6, num_local_experts=experts, num_experts_per_tok=top,
                           intermediate_size=ff, routed_scaling_factor=1.0, norm_topk_prob=True, tie_word_embeddings=False,
                           max_position_embeddings=2 * CONTEXT)


def givozen_work(cfg, rows: int):
    """(weights a step of `rows` rows multiplies a row by, weights it must read), both in elements, summed over the layer
    runs (a repeated layer counts each time it runs); of routed experts a row uses `top` and a step reads at most rows x top."""
    used = read = 0.0
    for i, _, _ in cfg.passes():
        layer = cfg.layers[i]
        a = layer.mixer
        attention = cfg.width * (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim) + a.heads) + a.heads * a.vdim * cfg.width
        used += attention
        read += attention
        mlp = layer.mlp
        if mlp is None:
            continue
        if mlp.kind == "dense":
            used += 2 * cfg.width * mlp.ff
            read += 2 * cfg.width * mlp.ff
            continue
        fixed = cfg.width * mlp.experts + (3 * cfg.width * mlp.shared.ff + cfg.width if mlp.shared else 0)
        used += fixed + mlp.top * 3 * cfg.width * mlp.ff
        read += fixed + min(mlp.experts, rows * mlp.top) * 3 * cfg.width * mlp.ff
    return used, read


# name -> (width, layers, heads, kv heads, window, chunk, memory heads (of 128 x 128), dense ff, experts, picks, expert ff, vocab)
SALIPEL_SIZES = {
    "w2048": (2048, 8, 16, 4, 1024, 1024, 4, 8192, 8, 2, 2048, 32768),
    "w4096": (4096, 4, 32, 8, 1024, 1024, 8, 16384, 8, 2, 4096, 32768),
    "w256": (256, 4, 2, 1, 64, 48, 1, 768, 4, 2, 128, 1024),
}


def salipel_config(width, layers, heads, kv_heads, window, chunk, mem_heads, dense_ff, experts, top, ff, vocab):
    from llmx_amd.config.givozen import WavelengthScaling
    from llmx_amd.config.salipel import (ChunkAttentionConfig, DifferenceAttentionConfig, LayerConfig, MemoryConfig, MLPConfig, ParallelConfig,
                                         Rotation, SalipelConfig, WindowAttentionConfig)
    rot = Rotation(1e6, 64, WavelengthScaling(8.0, 1.0, 4.0, 8192.0))
    two = DifferenceAttentionConfig(heads=heads, kv_heads=kv_heads, dim=64, vdim=128, scale=64 ** -0.5, softcap=50.0, diff=0.3, rot=rot)
    side = ParallelConfig(WindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5, window=window, keep_first=4, rot=rot),
                          MemoryConfig(heads=mem_heads, dim=128, vdim=128, gate_cap=15.0), 1.0, 0.5)
    chunks = ChunkAttentionConfig(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5, chunk=chunk)
    dense, moe = MLPConfig("dense", dense_ff), MLPConfig("moe", ff, experts=experts, top=top, scale=2.0)
    kinds = [("attention_2", two, dense), ("attention_2", two, moe), ("parallel", side, dense), ("attention", chunks, moe)]
    return SalipelConfig(vocab=vocab, width=width, norm_eps=1e-6, residual_mult=0.7, layers=tuple(LayerConfig(*kinds[i % 4]) for i in range(layers)))


def salipel_closest(width, layers, heads, kv_heads, window, chunk, mem_heads, dense_ff, experts, top, ff, vocab):
    """MiniMax-M3 of the same width, layers, heads, head width, experts, picks and expert width."""
    return bonerax_closest(width, layers, heads, kv_heads, window, mem_heads, experts, top, ff, vocab)


def salipel_work(cfg, rows: int):
    """(weights a step of `rows` rows multiplies a row by, weights it must read), both in elements; of routed experts a row
    uses `top` and a step reads at most rows x top."""
    used = read = 0.0
    E = cfg.width
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "attention":
            mix = E * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + m.heads * m.vdim * E
        elif layer.type == "attention_2":
            mix = E * (2 * m.heads * m.dim + m.kv_heads * (2 * m.dim + m.vdim) + m.heads * m.vdim) + m.heads * m.vdim * E
        else:
            a, b = m.left, m.right
            mix = E * (a.heads * a.dim + a.kv_heads * a.dim + a.heads * a.vdim) + a.heads * a.vdim * E
            mix += E * (2 * b.heads * b.dim + 2 * b.heads * b.vdim + 2 * b.heads) + b.heads * b.vdim * E
        used += mix
        read += mix
        mlp = layer.mlp
        if mlp is None:
            continue
        if mlp.kind == "dense":
            used += 3 * E * mlp.ff
            read += 3 * E * mlp.ff
        else:
            used += E * mlp.experts + mlp.top * 2 * E * mlp.ff
            read += E * mlp.experts + min(mlp.experts, rows * mlp.top) * 2 * E * mlp.ff
    return used, read


def salipel_mixing_flops(cfg, T: int) -> float:
    """Multiply-adds x 2 of the mixers' own work over a T-token prompt: scores and value products over the keys a row sees
    (twice the scores for two maps, and two value products), and the matrix memory's decay, outer product and read-out."""
    total = 0.0
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "attention":
            keys = sum(t % m.chunk + 1 for t in range(T))
            total += 2.0 * m.heads * (m.dim + m.vdim) * keys
        elif layer.type == "attention_2":
            total += 2.0 * m.heads * 2 * (m.dim + m.vdim) * T * (T + 1) / 2
        else:
            a, b = m.left, m.right
            keys = sum(min(t + 1, a.window) + min(a.keep_first, max(0, t + 1 - a.window)) for t in range(T))
            total += 2.0 * a.heads * (a.dim + a.vdim) * keys
            total += T * b.heads * b.dim * (b.vdim + 1) * 5.0
    return total


def _layer_mixers(layer):
    """(windowed attention or None, [recurrences as (heads, dim, vdim, delta?)]) of a Bonerax layer."""
    m = layer.mixer
    if layer.type == "parallel":
        return m.left, [(m.right.heads, m.right.dim, m.right.vdim, True)]
    return None, [(m.heads, m.dim, m.vdim, layer.type == "channel_delta")]


def _ids(n, vocab, seed):
    x, out = (seed * 2654435761 + 1) & 0xFFFFFFFF, []
    for _ in range(n):
        x = (x * 1664525 + 1013904223) & 0xFFFFFFFF
        out.append((x >> 8) % vocab)
    return out


def cache_bytes_a_token(engine) -> int:
    """Bytes of paged cache one token of one request holds over all layers."""
    return sum(t.shape[0] * (t.numel() // (t.shape[0] * t.shape[1]) // engine.page_tokens) * t.element_size()
               for arenas in engine._paged for t in arenas.values())


def cache_bytes_read(engine, context: float) -> float:
    """Bytes of cache and state a decoded token of one request at `context` tokens must read (and, for states, write):
    a windowed group's keys and values only as far as the window reaches."""
    total = 0.0
    for need, arenas in zip(engine.group_needs, engine._paged):
        tokens = min(context, need.window + getattr(need, "keep_first", 0)) if need.window else context
        if getattr(need, "chunk", None):
            tokens = min(tokens, need.chunk / 2.0)      # a decoded row sits anywhere in its chunk
        total += tokens * sum(t.shape[0] * (t.numel() // (t.shape[0] * t.shape[1]) // engine.page_tokens) * t.element_size() for t in arenas.values())
    return total + 2 * sum(t[0].numel() * t.element_size() for t in engine._state)


def prompt_flops(engine, T) -> float:
    """Multiply-adds x 2 of a T-token prompt: every weight matrix once a row (the head for one row), and the attention
    layers' score and value products over the causal half."""
    cfg = engine.config
    weights = sum(v.numel() for p in engine.model.parts() for v in vars(p).values()
                  if hasattr(v, "numel") and hasattr(v, "dim") and v.dim() >= 2 and v.dtype.is_floating_point)
    vocab = engine.spec.vocab_size
    dense = 2.0 * T * (weights - 2 * vocab * engine.spec.hidden_size) + 2.0 * vocab * engine.spec.hidden_size
    if hasattr(cfg, "num_local_experts"):      # only the picked experts work
        expert = 3 * cfg.hidden_size * cfg.intermediate_size
        dense -= 2.0 * T * cfg.num_hidden_layers * (cfg.num_local_experts - cfg.num_experts_per_tok) * expert
        attn = cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * T * (T + 1) / 2
    elif cfg.architecture == "Givozen":
        dense = 2.0 * T * givozen_work(cfg, T)[0] + 2.0 * vocab * engine.spec.hidden_size
        attn = sum(2.0 * cfg.layers[i].mixer.heads * (cfg.layers[i].mixer.dim + cfg.layers[i].mixer.vdim) * T * (T + 1) / 2 for i, _, _ in cfg.passes())
    elif cfg.architecture == "Salipel":
        dense = 2.0 * T * salipel_work(cfg, T)[0] + 2.0 * vocab * engine.spec.hidden_size
        attn = salipel_mixing_flops(cfg, T)
    elif cfg.architecture == "Bonerax":
        attn = 0.0
        for layer in cfg.layers:
            if layer.mlp is not None and layer.mlp.kind == "moe":
                dense -= 2.0 * T * (layer.mlp.experts - layer.mlp.top) * 3 * cfg.width * layer.mlp.ff
            left, recurrences = _layer_mixers(layer)
            if left is not None:
                keys = sum(min(t + 1, left.window) for t in range(T))
                attn += 2.0 * left.heads * (left.dim + left.vdim) * keys
            for heads, dim, vdim, delta in recurrences:      # decay, (S^T k,) the outer product, S^T q: a token a head
                attn += T * heads * dim * vdim * (2.0 * (3 if delta else 2) + 1.0)
    else:
        attn = 0.0
        for layer in cfg.layers:
            if layer.type == "latent_attention":
                m = layer.mixer
                attn += 2.0 * m.heads * (2 * m.kv_rank + m.rot_dim) * T * (T + 1) / 2     # over the latents themselves
                dense -= 0.0
        side = getattr(cfg, "token_side_dim", None) or 0
        dense -= 2.0 * T * vocab * side * len(cfg.layers)                                   # the token table is read, not multiplied
    return dense + attn


def measure(engine, torch, steps, warmup):
    from llmx_amd import ops
    from llmx_amd.engine import StepEntry
    vocab = engine.spec.vocab_size
    out = torch.empty(8, dtype=torch.int32, device=engine.device)
    rec = {"weights_gb": round(engine.weight_bytes() / 1e9, 2)}
    times = []
    for rep in range(3):
        rid = f"p{rep}"
        engine.add_request(rid)
        ids = _ids(PROMPT, vocab, 500 + rep)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry(rid, ids, [PROMPT - 1])])
        ops.argmax_rows(logits, out[:1])
        out[:1].tolist()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.end_request(rid)
    t = min(times[1:])
    flops = prompt_flops(engine, PROMPT)
    rec.update(prefill_tok_s=round(PROMPT / t, 1), prefill_ms=round(t * 1e3, 3), prefill_tflop=round(flops / 1e12, 4),
               prefill_frac=round(flops / t / BF16_PEAK, 4))
    for batch in (1, 8):
        start = CONTEXT - steps - warmup
        rids = [f"d{batch}_{i}" for i in range(batch)]
        for i, rid in enumerate(rids):
            engine.add_request(rid)
            ids = _ids(start, vocab, 100 + i)
            for s in range(0, start, PROMPT):
                engine.step([StepEntry(rid, ids[s:s + PROMPT], [])])
        last = [_ids(1, vocab, 7 + i)[0] for i in range(batch)]

        def one():
            nonlocal last
            logits = engine.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, last)])
            ops.argmax_rows(logits, out[:batch])
            last = out[:batch].tolist()

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        for rid in rids:
            engine.end_request(rid)
        need = engine.weight_bytes() + batch * cache_bytes_read(engine, CONTEXT - steps / 2)
        cfg = engine.config
        if hasattr(cfg, "num_local_experts"):   # of the experts at most batch x picks are read
            unread = max(0, cfg.num_local_experts - batch * cfg.num_experts_per_tok)
            need -= cfg.num_hidden_layers * unread * 3 * cfg.hidden_size * cfg.intermediate_size * 2
        elif cfg.architecture == "Bonerax":
            for layer in cfg.layers:
                if layer.mlp is not None and layer.mlp.kind == "moe":
                    need -= max(0, layer.mlp.experts - batch * layer.mlp.top) * 3 * cfg.width * layer.mlp.ff * 2
        side = getattr(cfg, "token_side_dim", None) or 0
        need -= 2 * vocab * side * (len(cfg.layers) if side else 0)     # of the token table a step reads its rows only
        need -= 2 * vocab * engine.spec.hidden_size                     # and of the embedding
        if cfg.architecture == "Salipel":
            need = 2 * (salipel_work(cfg, batch)[1] + vocab * engine.spec.hidden_size) + batch * cache_bytes_read(engine, CONTEXT - steps / 2)
        if cfg.architecture == "Givozen":       # weights by layer run; the head is the embedding's table, read whole
            need = 2 * (givozen_work(cfg, batch)[1] + vocab * engine.spec.hidden_size) + batch * cache_bytes_read(engine, CONTEXT - steps / 2)
        rec.update({f"decode_b{batch}_tok_s": round(batch / dt, 2), f"decode_b{batch}_ms": round(dt * 1e3, 4),
                    f"decode_b{batch}_gb": round(need / 1e9, 3), f"decode_b{batch}_frac": round(need / dt / 1e9 / HBM_PEAK_GBS, 4)})
    return rec


DESIGNS = {
    "nenotar": ("Nenotar", "MiniMax-M3 (GQA attention, routed SwiGLU experts)", SIZES, nenotar_config, closest_config),
    "bonerax": ("Bonerax", "MiniMax-M3 (GQA attention, routed SwiGLU experts)", BONERAX_SIZES, bonerax_config, bonerax_closest),
    "givozen": ("Givozen", "MiniMax-M3 (GQA attention, routed SwiGLU experts)", GIVOZEN_SIZES, givozen_config, givozen_closest),
    "salipel": ("Salipel", "MiniMax-M3 (GQA attention, routed SwiGLU experts)", SALIPEL_SIZES, salipel_config, salipel_closest),
}


def run(design: str, steps: int, warmup: int, sizes=None) -> dict:
    import torch
    from llmx_amd import Engine, RandomInit
    if design not in DESIGNS:
        raise SystemExit(f"bench: no design named {design!r} (known: {sorted(DESIGNS)})")
    title, closest, table, make_design, make_closest = DESIGNS[design]
    result = {"design": title, "closest": closest, "dtype": "bf16", "prompt": PROMPT,
              "context": CONTEXT, "data": "synthetic: LCG token ids, N(0,0.02) weights generated on the device", "sizes": {}}
    for name in (sizes or DEFAULT_SIZES):
        if name not in table:
            raise SystemExit(f"bench: no size named {name!r} (known: {sorted(table)})")
        shape = table[name]
        per = {}
        for which, make in ((design, make_design), ("closest", make_closest)):
            engine = Engine.from_random(make(*shape), RandomInit(seed=0, std=0.02), dtype="bfloat16", kv_tokens=8 * CONTEXT + 4 * PROMPT,
                                        page_tokens=16, max_requests=8)
            per[which] = measure(engine, torch, steps, max(2, warmup))
            del engine
            torch.cuda.empty_cache()
        result["sizes"][name] = per
    return result


def main(design: str, steps: int, warmup: int, sizes=None) -> None:
    print(json.dumps(run(design, steps, warmup, sizes)))
