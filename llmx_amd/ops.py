"""Python face of the gfx950 kernel library.

Each function checks on the host that its operands are what the kernel and its
grid assume (device, dtype, contiguity, shapes, index ranges that the host
knows) and then launches on torch's current stream.  There is no CPU path: a
missing library or a tensor that is not on the GPU is an error.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Optional

import torch

from .csrc import build as _build
from .limits import MAX_EXPERTS, MAX_HEAD_DIM, MAX_TOP_K

F32, BF16 = 0, 1
EPI_STORE, EPI_ADD, EPI_SWIGLU = 0, 1, 2
QKNORM_NONE, QKNORM_PROJECTION, QKNORM_HEAD = 0, 1, 2
ROPE_HALVES, ROPE_INTERLEAVED = 0, 1        # a head's rotated pairs: (i, i + R/2) or (2i, 2i + 1)
SCORE_SIGMOID, SCORE_SOFTMAX = 0, 1


class KernelError(RuntimeError):
    pass


_lib = None


def lib():
    """The loaded kernel library; built at the first call when nothing is built."""
    global _lib
    if _lib is None:
        path = _build.load_path()
        try:
            handle = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelError(f"the kernel library {path} could not be loaded: {e}") from None
        _declare(handle)
        handle._path = str(path)
        _lib = handle
    return _lib


def library_path() -> str:
    return lib()._path


def _declare(h) -> None:
    P, I, F, L = c_void_p, c_int, c_float, c_long
    sigs = {
        "llmx_embed_gather": [P, I, P, P, I, I, F, P],
        "llmx_rmsnorm_pair": [P, P, P, F, P, P, I, I, I, P],
        "llmx_scale_add": [P, P, P, P, P, P, I, I, I, P],
        "llmx_rmsnorm_add": [P, P, P, F, I, I, P],
        "llmx_act_xielu": [P, P, P, I, L, P],
        "llmx_act_gelu_gather": [P, P, I, P, P, I, I, I, I, I, P],
        "llmx_mingru_scan": [P, P, P, P, P, P, P, P, I, I, I, P],
        "llmx_mingru_scan_chunks": [P, P, P, P, P, P, P, P, I, I, I, P, I, P, P, P, P],
        "llmx_latent_prep": [P, P, P, P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, I, I, I, P],
        "llmx_latent_attention_mfma": [P, P, P, P, P, P, P, P, I, I, I, P, I, P, P, P, F, I, I, I, I, I, I, P],
        "llmx_latent_attention_mfma_ok": [I, I, I],
        "llmx_latent_attention_generic": [P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, P],
        "llmx_head_gate": [P, P, I, P, I, I, I, I, P],
        "llmx_rmsnorm": [P, P, P, F, P, I, P, I, I, P],
        "llmx_moe_combine": [P, P, P, P, I, I, I, I, P],
        "llmx_fill_i32": [P, I, L, P],
        "llmx_fill_random": [P, I, L, ctypes.c_ulonglong, I, F, F, P],
        "llmx_read_probe": [P, L, P, P],
        "llmx_attention_partial_pad": [],
        "llmx_gemm_generic": [P, I, P, I, P, I, I, I, I, I, I, I, I, I, P, P, I, L, I, I, P, I, F, P, P, I, P],
        "llmx_qknorm_rope_kvwrite": [P, P, P, P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, I, I, I, P],
        "llmx_paged_attention_generic": [P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, I, P, I, I, I, I, I, F, P, P, I, P],
        "llmx_head_norm_rope_kvwrite": [P, P, P, P, P, P, P, P, P, P, P, I, F, I, I, I, I, I, I, I, I, I, I, I, P, I, I, I, I, P],
        "llmx_gate_heads": [P, I, P, I, I, I, I, P],
        "llmx_rmsnorm_add_norm": [P, P, P, F, P, F, P, I, P, I, I, P],
        "llmx_add_rows_vector": [P, P, P, I, I, P],
        "llmx_act_polynorm": [P, P, F, P, I, I, I, P],
        "llmx_act_glu": [P, I, P, P, I, I, F, P, I, I, I, P],
        "llmx_layernorm": [P, P, P, F, P, I, P, I, I, P],
        "llmx_layernorm_add": [P, P, P, F, P, I, I, I, P],
        "llmx_cast_rows": [P, P, I, L, P],
        "llmx_combine_rows": [P, P, F, P, P, F, I, I, I, P],
        "llmx_scale_softcap": [P, F, F, L, P],
        "llmx_delta_prep": [P, I, P, P, I, P, P, P, L, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P],
        "llmx_cast_cols": [P, I, P, I, I, I, P],
        "llmx_sigmoid_root": [P, P, F, P, I, I, P],
        "llmx_state_scan": [P, I, P, I, P, I, P, I, P, P, L, P, P, P, P, F, I, I, I, I, I, P, I, I, I, I, I, P],
        "llmx_head_norm_gate": [P, P, P, I, P, I, F, I, I, I, I, I, I, I, F, F, P, P],
        "llmx_attention_rules": [P, P, P, P, P, P, P, I, P, I, P, I, P, I, P, P, F, F, I, I, I, I, I, I, I, I, I, I, P, P, P, I, I, I, P],
        "llmx_attention_rules_shared_ok": [I, I],
        "llmx_attention_rules_ok": [I, I, I, I],
        "llmx_attention_rules_segment": [],
        "llmx_memory_prep": [P, I, I, I, I, I, P, P, F, P, L, I, P, P, P, P, P, P, P, P, I, I, I, I, I, P],
        "llmx_paged_attention_mfma": [P, P, P, P, P, P, P, I, I, I, P, I, P, P, P, F, I, I, I, I, I, I, I, P, I, P],
        "llmx_route_topk": [P, P, I, L, P, P, P, I, I, I, I, I, F, P, P],
        "llmx_moe_align": [P, I, I, P, P, P, P, P, P, P, P],
        "llmx_route_topk_align": [P, P, I, L, P, P, P, I, I, I, I, F, P, P, P, P, P, P],
        "llmx_gemm_skinny": [P, P, P, I, I, I, I, I, I, I, I, I, I, P, P, P, P, I, L, I, P, P, F, I, I, P, I, F, P, P, I, P],
        "llmx_gemm_skinny_normed_ok": [I, I],
        "llmx_gemm_skinny_f32_normed_ok": [I, I],
        "llmx_argmax_rows": [P, P, P, P, I, I, P],
        "llmx_gemm_skinny_f32": [P, P, P, I, I, I, I, I, I, I, I, L, P, F, P],
        "llmx_gemm_tile": [P, P, P, I, I, I, I, I, I, I, I, I, I, P, P, I, L, I, P, P, I, P, I, F, P, P, I, P],
        "llmx_gemm_tile_offsets_fit": [I, I, I, I, I, I, I, I],
        "llmx_sample_all": [P, P, P, P, P, P, I, I, P, P],
        "llmx_sample_topk": [P, P, P, P, P, P, P, P, I, I, P, I, P],
        "llmx_sample_ranked": [P, P, P, P, P, P, P, P, I, I, P, P],
        "llmx_penalize": [P, P, P, P, P, P, P, I, I, P],
    }
    sigs.update({"llmx_note_launch": [I], "llmx_launch_kinds": [], "llmx_launch_name": [I], "llmx_take_launches": [P, I]})
    for name, args in sigs.items():
        try:
            fn = getattr(h, name)
        except AttributeError:
            raise KernelError(f"the kernel library lacks {name}; build it again from the current sources") from None
        fn.argtypes = args
        fn.restype = c_int
    h.llmx_sample_topk_scratch.argtypes = [I, I, I]
    h.llmx_sample_topk_scratch.restype = c_long
    h.llmx_sample_all_scratch.argtypes = [I, I]
    h.llmx_sample_all_scratch.restype = c_long
    h.llmx_sample_ranked_scratch.argtypes = [I, I]
    h.llmx_sample_ranked_scratch.restype = c_long
    h.llmx_gemm_tile_runs_scratch.argtypes = [I, I, I, I, I, I]
    h.llmx_gemm_tile_runs_scratch.restype = c_long
    h.llmx_launch_name.restype = ctypes.c_char_p
    h.llmx_note_launch.restype = None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (asked for at every launch, so through torch's raw accessor where it has one)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


def _dev(t: Optional[torch.Tensor], name: str, dtype=None, shape=None) -> int:
    """Checks a kernel operand and returns its address (0 for None)."""
    if t is None:
        return 0
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU (there is no CPU path)")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, not {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.data_ptr()


def _check(rc: int, what: str) -> None:
    if rc == -2:
        raise KernelError(f"{what}: a size this kernel does not take")
    if rc != 0:
        raise KernelError(f"{what}: launch failed with HIP error {rc}")


def launch_kinds() -> list:
    """The names under which the library counts its launches: one for every kernel form of every entry point."""
    h = lib()
    return [h.llmx_launch_name(i).decode() for i in range(h.llmx_launch_kinds())]


def take_launches() -> dict:
    """Which kernel forms were launched since the last call, by name, with their counts (forms that were not are
    left out); the counts are cleared.  The library counts on the host at every launch site, so this tells a test which
    of several kernels with equal results ran (/root/reference/src/backends/backend.hpp:96-112 keeps such a record for
    the same purpose).  A launch recorded into a HIP graph counts once, at the recording, not at replays."""
    h = lib()
    n = h.llmx_launch_kinds()
    counts = (c_long * n)()
    h.llmx_take_launches(counts, n)
    return {h.llmx_launch_name(i).decode(): int(counts[i]) for i in range(n) if counts[i]}


# ---------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = table[ids[t]] * scale, widened to float32."""
    rows, width = out.shape
    _check(lib().llmx_embed_gather(_dev(table, "table", shape=(table.shape[0], width)), _code(table.dtype),
                                   _dev(ids, "ids", torch.int32, (rows,)), _dev(out, "out", torch.float32),
                                   rows, width, float(scale), _stream()), "embed_gather")


def rmsnorm_pair(x: torch.Tensor, w1: torch.Tensor, w2: Optional[torch.Tensor], eps: float, out1: torch.Tensor,
                 out2: Optional[torch.Tensor]) -> None:
    """Two RMS norms of the same float32 rows with one eps and two gains: out1 = x * (r * w1), out2 = x * (r * w2), r formed
    once; each output has the bits `rmsnorm` gives with its gain."""
    rows, n = x.shape
    if (w2 is None) != (out2 is None) or (out2 is not None and out2.dtype != out1.dtype):
        raise KernelError("rmsnorm_pair: the second gain and the second output come together, in the first output's type")
    _check(lib().llmx_rmsnorm_pair(_dev(x, "x", torch.float32), _dev(w1, "w1", torch.float32, (n,)), _dev(w2, "w2", torch.float32, (n,)),
                                   float(eps), _dev(out1, "out1", shape=(rows, n)), _dev(out2, "out2", shape=(rows, n)), _code(out1.dtype),
                                   rows, n, _stream()), "rmsnorm_pair")


def scale_add(x: torch.Tensor, y1: torch.Tensor, s1: Optional[torch.Tensor], y2: Optional[torch.Tensor] = None,
              s2: Optional[torch.Tensor] = None, copy: Optional[torch.Tensor] = None) -> None:
    """x += s1 * y1 (+ s2 * y2), float32 rows and per-feature scales (None: 1); `copy` receives the new rows in its type."""
    rows, n = x.shape
    _check(lib().llmx_scale_add(_dev(x, "x", torch.float32), _dev(y1, "y1", torch.float32, (rows, n)), _dev(s1, "s1", torch.float32, (n,)),
                                _dev(y2, "y2", torch.float32, (rows, n)), _dev(s2 if y2 is not None else None, "s2", torch.float32, (n,)),
                                _dev(copy, "copy", shape=(rows, n)), _code(copy.dtype) if copy is not None else F32, rows, n, _stream()),
           "scale_add")


def rmsnorm_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """x += RMSNorm(y) * weight, all float32."""
    rows, n = x.shape
    _check(lib().llmx_rmsnorm_add(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, (rows, n)), _dev(weight, "weight", torch.float32, (n,)),
                                  float(eps), rows, n, _stream()), "rmsnorm_add")


def add_rows_vector(x: torch.Tensor, rows: Optional[torch.Tensor], vec: Optional[torch.Tensor]) -> None:
    """x[t] = (x[t] + rows[t]) + vec, float32; rows [T, n] and vec [n] may each be None."""
    T, n = x.shape
    _check(lib().llmx_add_rows_vector(_dev(x, "x", torch.float32), _dev(rows, "rows", torch.float32, (T, n)), _dev(vec, "vec", torch.float32, (n,)),
                                      T, n, _stream()), "add_rows_vector")


def act_polynorm(z: torch.Tensor, abce: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = a U(z) + b U(z^2) + c U(z^3) + e over float32 rows z [T, n], U(v) = v / sqrt(mean(v^2) + eps) a row, powers
    element by element; abce = (a, b, c, e) float32 on the device."""
    rows, n = z.shape
    _check(lib().llmx_act_polynorm(_dev(z, "z", torch.float32), _dev(abce, "abce", torch.float32, (4,)), float(eps),
                                   _dev(out, "out", shape=(rows, n)), _code(out.dtype), rows, n, _stream()), "act_polynorm")


GLU_SILU, GLU_CLAMPED, GLU_GELU_TANH = 0, 1, 2


class Glu:
    """The gated unit of a product's gated epilogue (EPI_SWIGLU) or of `act_glu`.  kind GLU_SILU: silu(gate) * up; GLU_CLAMPED:
    g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1); GLU_GELU_TANH: the tanh form of gelu(gate) * up.  row_scale (float32 [rows of c]; None: 1):
    a factor on both pre-activations of a row (a weight on what the product reads, the product being linear); row_gate (a
    float32 view [rows of c, 1], rows possibly strided; None: none): the row's result is multiplied by sigmoid(row_gate)."""

    def __init__(self, kind: int = GLU_SILU, limit: float = 0.0, row_scale: Optional[torch.Tensor] = None,
                 row_gate: Optional[torch.Tensor] = None):
        if kind not in (GLU_SILU, GLU_CLAMPED, GLU_GELU_TANH) or (kind == GLU_CLAMPED and not limit > 0.0):
            raise KernelError("a gated unit is GLU_SILU, GLU_CLAMPED or GLU_GELU_TANH, the clamped one with a positive limit")
        self.kind, self.limit, self.row_scale, self.row_gate = int(kind), float(limit), row_scale, row_gate

    @property
    def plain(self) -> bool:
        return self.kind == GLU_SILU and self.row_scale is None and self.row_gate is None

    def args(self, rows: int):
        """The five values the product kernels take, checked against the `rows` rows of c."""
        gate_at, gate_ld = _rows_view(self.row_gate, "row_gate", rows, 1) if self.row_gate is not None else (0, 0)
        return self.kind, self.limit, _dev(self.row_scale, "row_scale", torch.float32, (rows,)), gate_at, gate_ld


_NO_GLU = (0, 0.0, 0, 0, 0)
GLU_IN_EPILOGUE = True      # False: a product with another unit than silu(gate) * up stores its pre-activations and the unit's own kernel follows


def act_glu(pre: torch.Tensor, glu: Glu, out: torch.Tensor) -> None:
    """out[p] = unit(s gate, s up) (* sigmoid(row_gate[p])), where row p of the float32 `pre` [P, >= 2n] holds n gate values,
    then n up values, and s = glu.row_scale[p]: the gated unit as a kernel of its own."""
    P, n = out.shape
    if pre.dim() != 2 or pre.shape[0] != P or pre.shape[1] < 2 * n:
        raise KernelError(f"act_glu: pre-activations {tuple(pre.shape)} do not hold {P} rows of {n} gate and {n} up values")
    gate_at, gate_ld = _rows_view(glu.row_gate, "row_gate", P, 1) if glu.row_gate is not None else (0, 0)
    _check(lib().llmx_act_glu(_dev(pre, "pre", torch.float32), pre.shape[1], _dev(glu.row_scale, "row_scale", torch.float32, (P,)),
                              gate_at, gate_ld, glu.kind, glu.limit, _dev(out, "out"), _code(out.dtype), P, n, _stream()), "act_glu")


def rmsnorm_add_norm(x: torch.Tensor, y: torch.Tensor, w_join: torch.Tensor, eps_join: float, w_next: torch.Tensor, eps_next: float,
                     out: Optional[torch.Tensor], out32: Optional[torch.Tensor] = None) -> None:
    """x += RMSNorm(y) * w_join, then out / out32 = RMSNorm(x) * w_next of the new rows: a sublayer's normed result joined
    into the residual and the next sublayer's norm in one launch.  x, y float32 [T, n]; out in its own type, out32 float32."""
    rows, n = x.shape
    if out is None and out32 is None:
        raise KernelError("rmsnorm_add_norm needs an output")
    _check(lib().llmx_rmsnorm_add_norm(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, (rows, n)), _dev(w_join, "w_join", torch.float32, (n,)),
                                       float(eps_join), _dev(w_next, "w_next", torch.float32, (n,)), float(eps_next),
                                       _dev(out, "out", shape=(rows, n)), _code(out.dtype) if out is not None else F32,
                                       _dev(out32, "out32", torch.float32, (rows, n)), rows, n, _stream()), "rmsnorm_add_norm")


def act_xielu(z: torch.Tensor, pq: torch.Tensor, out: torch.Tensor) -> None:
    """out = xIELU(z) with the two numbers pq = (p, q) on the device: z > 0: softplus(p) z^2 + z/2; else (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    if out.shape != z.shape:
        raise KernelError("act_xielu: shapes do not agree")
    _check(lib().llmx_act_xielu(_dev(z, "z", torch.float32), _dev(pq, "pq", torch.float32, (2,)), _dev(out, "out"), _code(out.dtype),
                                z.numel(), _stream()), "act_xielu")


def act_gelu_gather(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, col0: int) -> None:
    """out[t, j] = gelu_tanh(z[t, j]) * table[ids[t], col0 + j]."""
    rows, n = z.shape
    if col0 < 0 or col0 + n > table.shape[1]:
        raise KernelError(f"act_gelu_gather: columns {col0}..{col0 + n} outside the table's {table.shape[1]}")
    _check(lib().llmx_act_gelu_gather(_dev(z, "z", torch.float32), _dev(table, "table"), _code(table.dtype), _dev(ids, "ids", torch.int32, (rows,)),
                                      _dev(out, "out", shape=(rows, n)), _code(out.dtype), rows, n, int(col0), table.shape[1], _stream()),
           "act_gelu_gather")


SCAN_CHUNK_ROWS = 64         # rows of a chunk of the recurrence's three-launch form
SCAN_CHUNKS_MIN_ROWS = 256   # an entry of at least this many rows in the step: the three-launch form runs


class ScanPlan:
    """The chunks of a step's rows for the recurrence's three-launch form (it holds no positions and no slots)."""

    def __init__(self, row_counts, device):
        import numpy as np
        chunks, per_entry, row0 = [], [], 0
        for e, n in enumerate(row_counts):
            first = len(chunks)
            for r in range(0, n, SCAN_CHUNK_ROWS):
                chunks.append([e, row0 + r, min(SCAN_CHUNK_ROWS, n - r), 1 if r + SCAN_CHUNK_ROWS >= n else 0])
            per_entry.append([first, len(chunks) - first])
            row0 += n
        self.n_chunks = len(chunks)
        self.chunks = torch.tensor(np.asarray(chunks, dtype=np.int32), device=device)
        self.entry_chunks = torch.tensor(np.asarray(per_entry, dtype=np.int32), device=device)


_SCAN_PLANS: dict = {}


def scan_plan(row_counts, device) -> Optional[ScanPlan]:
    """The chunk lists for a step with these rows an entry, or None when no entry is long enough for them to pay."""
    if max(row_counts) < SCAN_CHUNKS_MIN_ROWS:
        return None
    key = (tuple(row_counts), str(device))
    plan = _SCAN_PLANS.get(key)
    if plan is None:
        if len(_SCAN_PLANS) > 64:
            _SCAN_PLANS.clear()
        plan = _SCAN_PLANS[key] = ScanPlan(row_counts, device)
    return plan


def mingru_scan(zxg: torch.Tensor, bz: Optional[torch.Tensor], bx: Optional[torch.Tensor], state: torch.Tensor, slot_read: torch.Tensor,
                slot_write: torch.Tensor, entry_rows: torch.Tensor, out: torch.Tensor, plan: Optional[ScanPlan] = None, scratch=None) -> None:
    """The minGRU recurrence over each entry's rows (see csrc/recurrent.hip): zxg [T, 3W] float32 pre-activations
    (gate | candidate | output gate), state [slots, W] float32 read at slot_read[e] and written at slot_write[e],
    entry_rows [n_entries, 2] (first row, rows); out [T, W] = S_t * silu(g_t).  With a `plan` (scan_plan) the rows are
    worked on in chunks by three launches; `scratch(name, shape, dtype)` gives them storage."""
    T, W3 = zxg.shape
    W = W3 // 3
    n_e = entry_rows.shape[0]
    if W3 != 3 * W or state.shape[1] != W or tuple(out.shape) != (T, W):
        raise KernelError("mingru_scan: shapes do not agree")
    if plan is not None:
        if plan.entry_chunks.shape[0] != n_e:
            raise KernelError("mingru_scan: the plan does not fit the step's entries")
        if scratch is None:
            scratch = lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=zxg.device)
        chunk_a = scratch("scan.chunk_a", (plan.n_chunks, W), torch.float32)
        chunk_b = scratch("scan.chunk_b", (plan.n_chunks, W), torch.float32)
        _check(lib().llmx_mingru_scan_chunks(_dev(zxg, "zxg", torch.float32), _dev(bz, "bz", torch.float32, (W,)), _dev(bx, "bx", torch.float32, (W,)),
                                             _dev(state, "state", torch.float32), _dev(slot_read, "slot_read", torch.int32, (n_e,)),
                                             _dev(slot_write, "slot_write", torch.int32, (n_e,)), _dev(entry_rows, "entry_rows", torch.int32, (n_e, 2)),
                                             _dev(out, "out"), _code(out.dtype), n_e, W, _dev(plan.chunks, "chunks", torch.int32, (plan.n_chunks, 4)),
                                             plan.n_chunks, _dev(plan.entry_chunks, "entry_chunks", torch.int32, (n_e, 2)),
                                             _dev(chunk_a, "chunk_a"), _dev(chunk_b, "chunk_b"), _stream()), "mingru_scan_chunks")
        return
    _check(lib().llmx_mingru_scan(_dev(zxg, "zxg", torch.float32), _dev(bz, "bz", torch.float32, (W,)), _dev(bx, "bx", torch.float32, (W,)),
                                  _dev(state, "state", torch.float32), _dev(slot_read, "slot_read", torch.int32, (n_e,)),
                                  _dev(slot_write, "slot_write", torch.int32, (n_e,)), _dev(entry_rows, "entry_rows", torch.int32, (n_e, 2)),
                                  _dev(out, "out"), _code(out.dtype), n_e, W, _stream()), "mingru_scan")


def latent_prep(proj: torch.Tensor, norm_w: torch.Tensor, cos_sin: torch.Tensor, pos: torch.Tensor, row_entry: torch.Tensor,
                tables: torch.Tensor, q_plain: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, eps: float, heads: int, dim: int,
                rot_dim: int, rank: int, write_cache: bool = True, cache_t: Optional[torch.Tensor] = None) -> None:
    """From the float32 rows proj = [q of `heads` x (dim | rot_dim) | latent of `rank` | key part of rot_dim | ...]: the
    queries head by head (q_plain [H, T, dim], q_rot [H, T, rot_dim] rotated), and into the row's cache place the
    RMS-normed latent and the rotated key part.  cos_sin [positions, dims]: the first `dims` of a rotated part turn as
    interleaved pairs.  `cache_t` [pages, rank, page_tokens]: a second copy of the latent, transposed within the page."""
    T, ldp = proj.shape
    n_pages, page_tokens, width = cache.shape
    dims = cos_sin.shape[1]
    if cache_t is not None and (tuple(cache_t.shape) != (n_pages, rank, page_tokens) or cache_t.dtype != cache.dtype):
        raise KernelError("latent_prep: the transposed copy does not fit the cache")
    if width != rank + rot_dim or q_plain.dtype != cache.dtype or q_rot.dtype != cache.dtype:
        raise KernelError("latent_prep: the cache does not fit the latent and the key part")
    _check(lib().llmx_latent_prep(_dev(proj, "proj", torch.float32), _dev(norm_w, "norm_w", torch.float32, (rank,)),
                                  _dev(cos_sin, "cos_sin", torch.float32), _dev(pos, "pos", torch.int32, (T,)),
                                  _dev(row_entry, "row_entry", torch.int32, (T,)), _dev(tables, "tables", torch.int32),
                                  _dev(q_plain, "q_plain", shape=(heads, T, dim)), _dev(q_rot, "q_rot", shape=(heads, T, rot_dim)),
                                  _dev(cache, "cache"), _dev(cache_t, "cache_t"), _code(cache.dtype), float(eps), T, ldp, heads, dim, rot_dim, rank, dims, page_tokens,
                                  tables.shape[1], 1 if write_cache else 0, _stream()), "latent_prep")


def latent_attention(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, pos: torch.Tensor, row_entry: torch.Tensor,
                     tables: torch.Tensor, out: torch.Tensor, scale: float, window: int = 0, scratch=None,
                     cache_t: Optional[torch.Tensor] = None, plan: Optional["LatentPlan"] = None) -> None:
    """Causal softmax attention of every (head, row) over its request's paged latents: score = (q_lat . c + q_rot . k_rot)
    * scale, result = sum of weights * c.  q_lat and out [H, T, C], q_rot [H, T, R], cache [pages, page_tokens, C + R].
    `scratch(name, shape, dtype)`: storage that lives as long as the caller's step.  With `cache_t` (the latents once
    more, [pages, C, page_tokens]) and a `plan` (latent_plan) the matrix-core kernel runs, where latent_attention_mfma_ok
    says it can; otherwise the universal kernel."""
    H, T, C = q_lat.shape
    R = q_rot.shape[2]
    n_pages, page_tokens, width = cache.shape
    if width != C + R or tuple(q_rot.shape[:2]) != (H, T) or out.shape != q_lat.shape or len({q_lat.dtype, q_rot.dtype, cache.dtype, out.dtype}) != 1:
        raise KernelError("latent_attention: shapes or dtypes do not agree")
    if cache_t is not None and plan is not None and window == 0 and latent_attention_mfma_ok(q_lat.dtype, C, R, page_tokens):
        if plan.heads != H or plan.rows != T or tuple(cache_t.shape) != (n_pages, C, page_tokens) or cache_t.dtype != cache.dtype:
            raise KernelError("latent_attention: the plan or the transposed copy does not fit the step")
        part_o = part_ml = None
        if plan.n_slots:
            if scratch is None:
                scratch = lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=q_lat.device)
            part_o = scratch("latent.part_o", (plan.n_slots, 16, C), torch.float32)
            part_ml = scratch("latent.part_ml", (plan.n_slots, 16, 2), torch.float32)
        _check(lib().llmx_latent_attention_mfma(_dev(q_lat, "q_lat"), _dev(q_rot, "q_rot"), _dev(cache, "cache"), _dev(cache_t, "cache_t"),
                                                _dev(pos, "pos", torch.int32, (T,)), _dev(row_entry, "row_entry", torch.int32, (T,)),
                                                _dev(tables, "tables", torch.int32), _dev(plan.items, "items", torch.int32), plan.n_items,
                                                plan.n_tile_items, plan.n_row_items, _dev(plan.merges, "merges", torch.int32), plan.n_merges, _dev(out, "out"),
                                                _dev(part_o, "part_o"), _dev(part_ml, "part_ml"), float(scale), T, H, C, R, page_tokens,
                                                tables.shape[1], _stream()),
               "latent_attention_mfma")
        return
    _check(lib().llmx_latent_attention_generic(_dev(q_lat, "q_lat"), _dev(q_rot, "q_rot"), _dev(cache, "cache"), _dev(pos, "pos", torch.int32, (T,)),
                                               _dev(row_entry, "row_entry", torch.int32, (T,)), _dev(tables, "tables", torch.int32),
                                               _dev(out, "out"), _code(q_lat.dtype), float(scale), T, H, C, R, page_tokens, tables.shape[1],
                                               int(window), _stream()), "latent_attention")


def latent_attention_mfma_ok(dtype: torch.dtype, rank: int, rot_dim: int, page_tokens: int) -> bool:
    return dtype == torch.bfloat16 and bool(lib().llmx_latent_attention_mfma_ok(int(rank), int(rot_dim), int(page_tokens)))


LATENT_SPLIT_KEYS = 128    # keys a split item of a decoded row takes (two segments of the kernel)


class LatentPlan:
    """Work items of the matrix-core latent attention for one step's rows: each up to 16 (row, head) columns of one request,
    whole or, for decoded rows, one block of the context; and the list of joins of the split ones.  It holds no positions."""

    def __init__(self, tiles, row_items, items, merges, n_slots, heads, rows, device):
        import numpy as np
        self.heads, self.rows, self.n_items, self.n_merges, self.n_slots = heads, rows, len(items), len(merges), n_slots
        self.n_tile_items = len(tiles)       # the list's first items: four column tiles each, for a workgroup of four waves
        self.n_row_items = len(row_items)    # then the decoded rows' items: one column tile, a workgroup of four waves
        items = tiles + row_items + items
        self.items = torch.tensor(np.asarray(items, dtype=np.int32).reshape(-1, 8), device=device)
        self.merges = torch.tensor(np.asarray(merges, dtype=np.int32).reshape(-1, 8), device=device) if merges else None


_LATENT_PLANS: dict = {}


LATENT_TILES = 4           # column tiles of 16 that a workgroup of the prompt form takes (the kernel's LW_TILES)


def latent_plan(row_counts, heads: int, device, contexts=None, tiles: bool = True) -> LatentPlan:
    """row_counts[i]: rows of entry i (entries' rows are consecutive, in order); contexts[i]: the tokens it holds after the
    step (None: nothing is split).  With 16 heads or more an item is one row and up to 16 of its heads; with fewer,
    16 // heads consecutive rows of one entry with all their heads; later rows (longer key ranges) come first.  An entry of
    one row (a decoded token) whose context is longer than LATENT_SPLIT_KEYS gets an item for every block of that many
    keys, a function of its own context only.  An entry of several rows (a prompt's portion) goes, `tiles` allowing, to
    workgroups of four waves that take four column tiles each and read the keys once for all of them; the same bits."""
    blocks = tuple(-(-c // LATENT_SPLIT_KEYS) if n == 1 else 1 for n, c in zip(row_counts, contexts)) if contexts is not None else None
    key = (tuple(row_counts), heads, blocks, bool(tiles), str(device))
    plan = _LATENT_PLANS.get(key)
    if plan is None:
        wide, single, items, merges, row0, slot = [], [], [], [], 0, 0
        per = max(1, 16 // heads)
        for i, n in enumerate(row_counts):
            nb = blocks[i] if blocks is not None else 1
            if n <= 0:
                continue
            if tiles and n > per:      # more rows than one column tile holds
                span = per * LATENT_TILES
                for r in range(((n - 1) // span) * span, -1, -span):
                    for h0 in range(0, heads, 16):
                        wide.append([row0 + r, min(span, n - r), h0, min(16, heads - h0), 0, 0, -1, 0])
                row0 += n
                continue
            for r in range(((n - 1) // per) * per, -1, -per):
                for h0 in range(0, heads, 16):
                    nh = min(16, heads - h0)
                    to = single if (tiles and n == 1) else items      # a decoded row's items go to workgroups of four waves
                    if nb <= 1:
                        to.append([row0 + r, min(per, n - r), h0, nh, 0, 0, -1, 0])
                        continue
                    merges.append([row0, h0, nh, slot, nb, 0, 0, 0])
                    for b in range(nb):
                        to.append([row0, 1, h0, nh, b * LATENT_SPLIT_KEYS, (b + 1) * LATENT_SPLIT_KEYS, slot + b, 0])
                    slot += nb
            row0 += n
        if len(_LATENT_PLANS) > 256:
            _LATENT_PLANS.clear()
        plan = _LATENT_PLANS[key] = LatentPlan(wide, single, items, merges, slot, heads, row0, device)
    return plan


def head_gate(values: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[t, h*V + d] = sigmoid(gate[t, h]) * values[h, t, d]; gate a float32 view [T, H] whose rows may be strided
    (columns of a wider projection), or None for no gate."""
    H, T, V = values.shape
    ldg = 0
    addr = 0
    if gate is not None:
        if not gate.is_cuda or gate.dtype != torch.float32 or tuple(gate.shape) != (T, H) or gate.stride(1) != 1:
            raise KernelError("head_gate: the gate is float32 [T, H] on the GPU with unit stride along the heads")
        ldg, addr = gate.stride(0), gate.data_ptr()
    _check(lib().llmx_head_gate(_dev(values, "values", torch.float32), addr, ldg, _dev(out, "out", shape=(T, H * V)), _code(out.dtype),
                                T, H, V, _stream()), "head_gate")


_HEAD_GROUPS: dict = {}


def head_groups(heads: int, rows: int, device):
    """What grouped_gemm wants for `heads` groups of `rows` rows each, laid out group by group: (offsets, pairs, active,
    n_active) on the device.  Cached: a step's launches may be recorded into a graph that reads them later."""
    key = (heads, rows, str(device))
    got = _HEAD_GROUPS.get(key)
    if got is None:
        if len(_HEAD_GROUPS) > 512:
            _HEAD_GROUPS.clear()
        got = _HEAD_GROUPS[key] = (torch.arange(0, (heads + 1) * rows, rows, dtype=torch.int32, device=device),
                                   torch.arange(heads * rows, dtype=torch.int32, device=device),
                                   torch.arange(heads, dtype=torch.int32, device=device),
                                   torch.full((1,), heads, dtype=torch.int32, device=device))
    return got


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor], out32: Optional[torch.Tensor] = None,
            pick: Optional[torch.Tensor] = None) -> None:
    """out[r] = norm(x[pick[r]] or x[r]); out in its own dtype, out32 an optional float32 copy."""
    n = x.shape[-1]
    rows = pick.shape[0] if pick is not None else x.shape[0]
    if out is None and out32 is None:
        raise KernelError("rmsnorm needs an output")
    _check(lib().llmx_rmsnorm(_dev(x, "x", torch.float32), _dev(pick, "pick", torch.int32), _dev(weight, "weight", torch.float32, (n,)),
                              float(eps), _dev(out, "out", shape=(rows, n)), _code(out.dtype) if out is not None else F32,
                              _dev(out32, "out32", torch.float32, (rows, n)), rows, n, _stream()), "rmsnorm")


def layernorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor], out32: Optional[torch.Tensor] = None,
              pick: Optional[torch.Tensor] = None) -> None:
    """out[r] = (x - mean) / sqrt(var + eps) * weight of row x[pick[r]] (or x[r]), var the mean of the squared deviations;
    out in its own dtype, out32 an optional float32 copy."""
    n = x.shape[-1]
    rows = pick.shape[0] if pick is not None else x.shape[0]
    if out is None and out32 is None:
        raise KernelError("layernorm needs an output")
    _check(lib().llmx_layernorm(_dev(x, "x", torch.float32), _dev(pick, "pick", torch.int32), _dev(weight, "weight", torch.float32, (n,)),
                                float(eps), _dev(out, "out", shape=(rows, n)), _code(out.dtype) if out is not None else F32,
                                _dev(out32, "out32", torch.float32, (rows, n)), rows, n, _stream()), "layernorm")


def layernorm_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, copy: Optional[torch.Tensor] = None) -> None:
    """x += layer norm of y (weight, no bias), float32 rows; `copy` receives the new rows in its type."""
    rows, n = x.shape
    _check(lib().llmx_layernorm_add(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, (rows, n)), _dev(weight, "weight", torch.float32, (n,)),
                                    float(eps), _dev(copy, "copy", shape=(rows, n)), _code(copy.dtype) if copy is not None else F32, rows, n,
                                    _stream()), "layernorm_add")


def cast_rows(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = x (float32) in out's type."""
    if out.shape != x.shape:
        raise KernelError("cast_rows: shapes do not agree")
    _check(lib().llmx_cast_rows(_dev(x, "x", torch.float32), _dev(out, "out"), _code(out.dtype), x.numel(), _stream()), "cast_rows")


def cast_cols(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = x in out's type, x a float32 view [T, n] whose rows may be columns of a wider tensor."""
    rows, n = out.shape
    at, ld = _rows_view(x, "x", rows, n)
    _check(lib().llmx_cast_cols(at, ld, _dev(out, "out"), _code(out.dtype), rows, n, _stream()), "cast_cols")


def combine_rows(out: torch.Tensor, a: torch.Tensor, scale_a: float = 1.0, bias_a: Optional[torch.Tensor] = None,
                 b: Optional[torch.Tensor] = None, scale_b: float = 1.0, accumulate: bool = False) -> None:
    """out (= or +=) scale_a * (a + bias_a) + scale_b * b over float32 rows [T, n]; bias_a [n] and b may be None."""
    rows, n = out.shape
    _check(lib().llmx_combine_rows(_dev(out, "out", torch.float32), _dev(a, "a", torch.float32, (rows, n)), float(scale_a),
                                   _dev(bias_a, "bias_a", torch.float32, (n,)), _dev(b, "b", torch.float32, (rows, n)), float(scale_b),
                                   1 if accumulate else 0, rows, n, _stream()), "combine_rows")


def scale_softcap(z: torch.Tensor, scale: float, cap: float) -> None:
    """z <- z * scale, then cap * tanh(z / cap) when cap > 0; float32, in place."""
    _check(lib().llmx_scale_softcap(_dev(z, "z", torch.float32), float(scale), float(cap), z.numel(), _stream()), "scale_softcap")


def _rows_view(t: torch.Tensor, name: str, rows: int, cols: int):
    """(address, row stride) of a float32 [rows, cols] tensor whose rows may be columns of a wider one."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.float32 or tuple(t.shape) != (rows, cols) or (cols > 1 and t.stride(1) != 1):
        raise KernelError(f"{name} must be float32 [{rows}, {cols}] on the GPU with unit stride along a row")
    return t.data_ptr(), (t.stride(0) if rows > 1 else max(cols, t.stride(0)))


def delta_prep(pre: torch.Tensor, conv_w: torch.Tensor, step_pre: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
               state: torch.Tensor, tail_off: int, slot_read: torch.Tensor, row_entry: torch.Tensor, entry_rows: torch.Tensor,
               q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, beta: torch.Tensor, G: int, H: int, D: int, V: int,
               beta_col: int) -> None:
    """A delta-rule mixer's rows made ready for the scan (see csrc/linear_state.hip): from the fused in-projection `pre`
    [T, ld] = q (G*D) | k (G*D) | v (H*V) | ... | beta (H) at beta_col: the short causal convolution (conv_w [C, taps], the
    inputs of earlier steps from the state's tail at `tail_off`) with silu, unit-norm q and k heads, v, the decay
    exp(-exp(a_log) softplus(step_pre + dt_bias)) [T, H*D] and beta = sigmoid [T, H]."""
    T, ld = pre.shape
    C = 2 * G * D + H * V
    taps = conv_w.shape[1]
    n_e = entry_rows.shape[0]
    if state.dim() != 2 or tail_off + (taps - 1) * C > state.shape[1]:
        raise KernelError("delta_prep: the state does not hold the convolution's tail")
    step_at, step_ld = _rows_view(step_pre, "step_pre", T, H * D)
    _check(lib().llmx_delta_prep(_dev(pre, "pre", torch.float32), ld, _dev(conv_w, "conv_w", torch.float32, (C, taps)),
                                 step_at, step_ld, _dev(dt_bias, "dt_bias", torch.float32, (H * D,)),
                                 _dev(a_log, "a_log", torch.float32, (H,)), _dev(state, "state", torch.float32), state.shape[1], int(tail_off),
                                 _dev(slot_read, "slot_read", torch.int32, (n_e,)), _dev(row_entry, "row_entry", torch.int32, (T,)),
                                 _dev(entry_rows, "entry_rows", torch.int32, (n_e, 2)), _dev(q, "q", torch.float32, (T, G * D)),
                                 _dev(k, "k", torch.float32, (T, G * D)), _dev(v, "v", torch.float32, (T, H * V)),
                                 _dev(decay, "decay", torch.float32, (T, H * D)), _dev(beta, "beta", torch.float32, (T, H)),
                                 T, G, H, D, V, taps, int(beta_col), _stream()), "delta_prep")


def sigmoid_root(z: torch.Tensor, bias: Optional[torch.Tensor], tau: float, out: torch.Tensor) -> None:
    """out = sigmoid(z + bias)^(1 / tau), float32 [T, n]."""
    rows, n = z.shape
    _check(lib().llmx_sigmoid_root(_dev(z, "z", torch.float32), _dev(bias, "bias", torch.float32, (n,)), 1.0 / float(tau),
                                   _dev(out, "out", torch.float32, (rows, n)), rows, n, _stream()), "sigmoid_root")


STATE_TILE = 8      # value channels of a tile of a matrix state (the scan kernel's SCAN_COLS)


def state_matrix_size(H: int, D: int, V: int) -> int:
    """Floats a matrix state of H heads [D, V] takes in a state slot (its value channels padded to whole tiles)."""
    return H * -(-V // STATE_TILE) * D * STATE_TILE


def state_matrix_tiled(S: torch.Tensor) -> torch.Tensor:
    """A state [..., H, D, V] as the scan keeps it: [..., H * tiles * D * 8], value channel j of key channel d at tile j // 8,
    place d * 8 + j % 8 (zeros in the last tile's padding).  `state_matrix_plain` is its inverse."""
    *lead, H, D, V = S.shape
    tiles = -(-V // STATE_TILE)
    padded = torch.zeros(*lead, H, D, tiles * STATE_TILE, dtype=S.dtype, device=S.device)
    padded[..., :V] = S
    return padded.reshape(*lead, H, D, tiles, STATE_TILE).transpose(-3, -2).reshape(*lead, H * tiles * D * STATE_TILE)


def state_matrix_plain(flat: torch.Tensor, H: int, D: int, V: int) -> torch.Tensor:
    tiles = -(-V // STATE_TILE)
    lead = flat.shape[:-1]
    return flat[..., :H * tiles * D * STATE_TILE].reshape(*lead, H, tiles, D, STATE_TILE).transpose(-3, -2).reshape(*lead, H, D, tiles * STATE_TILE)[..., :V]


def state_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, beta: Optional[torch.Tensor], state: torch.Tensor,
               slot_read: torch.Tensor, slot_write: torch.Tensor, entry_rows: torch.Tensor, out: torch.Tensor, out_scale: float,
               H: int, qk_heads: int, D: int, V: int, tail=None, max_rows: int = 0) -> None:
    """The matrix-state recurrence over each entry's rows (csrc/linear_state.hip): per head S <- diag(decay) S;
    u = beta (v - S^T k) (u = v without beta); S <- S + k u^T; out = out_scale * S^T q.  q, k [T, qk_heads*D], v [T, H*V],
    decay [T, H*D] are float32 views whose rows may be columns of wider tensors; state [slots, width] float32 holds S at
    its start in tiles of 8 value channels ([H, ceil(V / 8), D, 8]: `state_matrix_size`, `state_matrix_tiled`), read at
    slot_read[e], written at slot_write[e].  `max_rows`: the most rows an entry has, when the caller knows it (steps of
    single tokens stage smaller chunks; the results are the same).  `tail` = (source [T, C] view, taps, offset):
    the convolution tail [taps - 1, C] at `offset` of the state is handed on from the step's rows of `source`."""
    T = out.shape[0]
    n_e = entry_rows.shape[0]
    if H % qk_heads or state.dim() != 2 or state.shape[1] < state_matrix_size(H, D, V) or D > 256:
        raise KernelError("state_scan: heads, widths or state do not fit")
    qa, ldq = _rows_view(q, "q", T, qk_heads * D)
    ka, ldk = _rows_view(k, "k", T, qk_heads * D)
    va, ldv = _rows_view(v, "v", T, H * V)
    ga, ldg = _rows_view(decay, "decay", T, H * D)
    ta, tld, tC, taps, toff = 0, 0, 0, 0, 0
    if tail is not None:
        src, taps, toff = tail
        tC = src.shape[1]
        ta, tld = _rows_view(src, "tail source", T, tC)
        if toff < state_matrix_size(H, D, V) or toff + (taps - 1) * tC > state.shape[1]:
            raise KernelError("state_scan: the state does not hold the convolution's tail")
    _check(lib().llmx_state_scan(qa, ldq, ka, ldk, va, ldv, ga, ldg, _dev(beta, "beta", torch.float32, (T, H)), _dev(state, "state", torch.float32),
                                 state.shape[1], _dev(slot_read, "slot_read", torch.int32, (n_e,)), _dev(slot_write, "slot_write", torch.int32, (n_e,)),
                                 _dev(entry_rows, "entry_rows", torch.int32, (n_e, 2)), _dev(out, "out", torch.float32, (T, H * V)), float(out_scale),
                                 n_e, H, H // qk_heads, D, V, ta, tld, tC, int(taps), int(toff), int(max_rows), _stream()), "state_scan")


GATE_SIGMOID, GATE_SILU = 0, 1


def head_norm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], gate_pre: Optional[torch.Tensor], out: torch.Tensor, eps: float, H: int, V: int,
                   gate: int, minus: Optional[float] = None, post: float = 1.0, den_floor: Optional[torch.Tensor] = None) -> None:
    """out[t, h] = x / sqrt(mean(x^2) + eps) * weight * gate(gate_pre[t, h]) * post for every head's V values x; gate is
    sigmoid or silu of a float32 view [T, H*V] (None: no gate); weight float32 [V] (one for all heads), [H*V], or None; out
    in its own type.  x is o's head [T, H*V]; with `minus` = lambda, o is [T, H*2*V], a head holding two maps, and
    x = map 1 - lambda * map 2; with `den_floor` (float32 [T, H]), o is [T, H*(V+1)], a head's values followed by their
    denominator d, and x = values / (max(|d|, den_floor) + 1e-6)."""
    T = o.shape[0]
    o_head = V * (2 if minus is not None else 1) + (1 if den_floor is not None else 0)
    if minus is not None and den_floor is not None:
        raise KernelError("head_norm_gate: a second map or a denominator, not both")
    za, ldz = _rows_view(gate_pre, "gate_pre", T, H * V) if gate_pre is not None else (0, 0)
    wide = 0
    if weight is not None:
        if tuple(weight.shape) not in ((V,), (H * V,)):
            raise KernelError(f"head_norm_gate: a weight of {V} or {H * V} values, not {tuple(weight.shape)}")
        wide = 1 if tuple(weight.shape) == (H * V,) and H > 1 else 0
    _check(lib().llmx_head_norm_gate(_dev(o, "o", torch.float32, (T, H * o_head)), _dev(weight, "weight", torch.float32), za, ldz,
                                     _dev(out, "out", shape=(T, H * V)), _code(out.dtype), float(eps), T, H, V, int(gate), o_head, wide,
                                     V if minus is not None else 0, float(minus or 0.0), float(post),
                                     _dev(den_floor, "den_floor", torch.float32, (T, H)), _stream()), "head_norm_gate")


def memory_prep(pre: torch.Tensor, cols: dict, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float, state: torch.Tensor, m_off: int,
                slot_read: torch.Tensor, slot_write: torch.Tensor, entry_rows: torch.Tensor, decay: torch.Tensor, keys: torch.Tensor,
                values: torch.Tensor, den_floor: torch.Tensor, H: int, D: int, V: int, factors: Optional[torch.Tensor] = None) -> None:
    """A gated matrix memory's rows made ready for `state_scan` (see csrc/linear_state.hip): from the fused projection `pre`
    [T, ld] with k (H*D), v (H*V) and the two gates' pre-activations (H each) at the columns cols["k"], ["v"], ["i"], ["f"]:
    i = cap tanh((zi + i_bias) / cap), f = log sigmoid(cap tanh((zf + f_bias) / cap)), the running maximum m = max(f + m, i)
    of each request (kept at `m_off` of its state slot, one float a head, read at slot_read, written at slot_write);
    decay [T, H*D] = exp(f + m_before - m), keys [T, H*D] = exp(i - m) k, values [T, H*(V+1)] = v | 1, den_floor [T, H] = exp(-m).
    `factors`: float32 [T, H, 2] of scratch (the rows' two factors on their way from the first launch to the second)."""
    T, ld = pre.shape
    if factors is None:
        factors = torch.empty((T, H, 2), dtype=torch.float32, device=pre.device)
    n_e = entry_rows.shape[0]
    if state.dim() != 2 or m_off + H > state.shape[1]:
        raise KernelError("memory_prep: the state does not hold the running maxima")
    if max(cols["k"] + H * D, cols["v"] + H * V, cols["i"] + H, cols["f"] + H) > ld:
        raise KernelError("memory_prep: the projection's rows do not hold the named columns")
    _check(lib().llmx_memory_prep(_dev(pre, "pre", torch.float32), ld, int(cols["k"]), int(cols["v"]), int(cols["i"]), int(cols["f"]),
                                  _dev(i_bias, "i_bias", torch.float32, (H,)), _dev(f_bias, "f_bias", torch.float32, (H,)), float(cap),
                                  _dev(state, "state", torch.float32), state.shape[1], int(m_off), _dev(slot_read, "slot_read", torch.int32, (n_e,)),
                                  _dev(slot_write, "slot_write", torch.int32, (n_e,)), _dev(entry_rows, "entry_rows", torch.int32, (n_e, 2)),
                                  _dev(decay, "decay", torch.float32, (T, H * D)), _dev(keys, "keys", torch.float32, (T, H * D)),
                                  _dev(values, "values", torch.float32, (T, H * (V + 1))), _dev(den_floor, "den_floor", torch.float32, (T, H)),
                                  _dev(factors, "factors", torch.float32, (T, H, 2)), T, n_e, H, D, V, _stream()), "memory_prep")


SKINNY_MAX_ROWS = 64          # dense products of at most this many rows stream the weights once on the matrix cores
TILE_RUNS_APART_MIN_ROWS = 17  # dense products from this many rows on take the tiled kernel with K's runs in workgroups of their own, where it offers that
SKINNY_WIDE_MAX_ROWS = 4      # ... and of at most this many rows however wide they are
TILE_FILL = 1024              # feature tiles of 128 from which the tiled kernel fills the chip with one tile of rows
SKINNY_MAX_GROUPED_ROWS = 16   # routed products of at most this many token rows do (measured: beyond it the tiled kernel streams the experts faster)


def _split_k(n_strips: int, K: int) -> int:
    """Runs the products cut K into (waves that share one 16-feature strip in the weight-streaming kernel; run boundaries
    in the tiled kernel): enough strips * runs to fill the chip, at least 12 steps of 32 a run.  A function of the
    product's shape only, so a row's bits do not depend on the batch."""
    ks = 1
    while ks < 8 and n_strips * ks < 2048 and (K // 32) // (ks * 2) >= 12:
        ks *= 2
    return ks


def _skinny_ok(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[-1] % 8 == 0
            and (epilogue != EPI_ADD or c.dtype == torch.float32))


class NormedRows:
    """The float32 rows x seen through an RMSNorm (weight, eps), not yet computed: a product that reads its rows this way
    forms norm(x) itself while its weights travel (steps of very few rows only), and no norm kernel runs."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float):
        self.x, self.weight, self.eps = x, weight, float(eps)
        self.shape = x.shape

    def args(self):
        return _dev(self.x, "x", torch.float32), _dev(self.weight, "norm weight", torch.float32, (self.x.shape[1],)), self.eps, self.x.shape[0]


_NO_NORM = (0, 0, 0.0, 0)


NORMED_ROWS_PAY = 1   # rows up to which a product that norms its own rows beats the norm kernel (measured: 1 row 3.07 -> 2.98 ms a step,
                      # 2 rows 4.03 -> 4.23, 4 rows 6.01 -> 6.11: the rows are formed one after the other in every workgroup)


def gemm_can_norm_rows(rows: int, w: torch.Tensor, c_dtype: torch.dtype, epilogue: int = EPI_STORE, grouped: bool = False) -> bool:
    """Whether gemm / grouped_gemm can form `rows` normed rows itself for this product (the weight-streaming kernel runs
    and the rows fit its LDS)."""
    K = w.shape[-1]
    return (w.dtype == torch.bfloat16 and epilogue != EPI_ADD and K % 8 == 0 and bool(lib().llmx_gemm_skinny_normed_ok(rows, K))
            and (grouped and rows <= SKINNY_MAX_GROUPED_ROWS or not grouped))


def gemm_f32_can_norm_rows(rows: int, w: torch.Tensor) -> bool:
    return bool(lib().llmx_gemm_skinny_f32_normed_ok(rows, w.shape[1]))


def gemm_takes_normed_rows(rows: int, w: torch.Tensor, c_dtype: torch.dtype, epilogue: int = EPI_STORE, grouped: bool = False) -> bool:
    """What a part answers a block that offers a deferred norm: the product can form the rows, and for so few rows that
    it pays."""
    return rows <= NORMED_ROWS_PAY and gemm_can_norm_rows(rows, w, c_dtype, epilogue, grouped)


def gemm_f32_takes_normed_rows(rows: int, w: torch.Tensor) -> bool:
    return rows <= NORMED_ROWS_PAY and gemm_f32_can_norm_rows(rows, w)


ACT_NONE, ACT_XIELU, ACT_RELU2 = 0, 1, 2      # activations a storing product can apply to what it stores (RELU2: max(z, 0)^2, no numbers)


def _act_args(act, epilogue: int, what: str):
    """The two values the product kernels take for `act` = (kind, params or None)."""
    if act is None:
        return 0, 0
    if epilogue != EPI_STORE or act[0] not in (ACT_XIELU, ACT_RELU2):
        raise KernelError(f"{what}: an activation goes with the store epilogue, and xIELU and the squared relu are the ones built")
    if act[0] == ACT_XIELU:
        return ACT_XIELU, _dev(act[1], "activation parameters", torch.float32, (2,))
    return ACT_RELU2, 0


def _scratch_now(device):
    """Storage for a caller that brings no step workspace: allocated at the call."""
    return lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=device)


def _glu_apart(glu: Optional["Glu"], epilogue: int) -> bool:
    """Whether a gated product runs as a storing product followed by the unit's own kernel."""
    if glu is None:
        return False
    if epilogue != EPI_SWIGLU:
        raise KernelError("a gated unit goes with the gated epilogue")
    return not glu.plain and not GLU_IN_EPILOGUE


def gemm(a, w: torch.Tensor, c: torch.Tensor, epilogue: int = EPI_STORE, force_generic: bool = False, scratch=None, act=None,
         glu: Optional["Glu"] = None) -> None:
    """c[M,N] (+)= a[M,K] @ w[N,K]^T, accumulated in float32; EPI_SWIGLU: c = silu(a @ w[:N]^T) * (a @ w[N:]^T).
    `a` may be NormedRows where gemm_takes_normed_rows says so: the product reads bfloat16(norm(x)).
    `scratch(name, shape, dtype)` gives storage that lives as long as the caller's step (a step's workspace): with it,
    products of some tens of rows multiply K's runs in workgroups of their own; the bits are the same either way.
    `act` = (ACT_XIELU, params) | (ACT_RELU2, None): with EPI_STORE, c = activation(a @ w^T), params the activation's
    numbers on the device (xIELU: float32 (p, q)); the bits of the product followed by the activation's own kernel (act_xielu).
    `glu`: the gated epilogue's unit (see Glu); None: silu(gate) * up."""
    M, K = a.shape
    if _glu_apart(glu, epilogue):
        if isinstance(a, NormedRows):
            raise KernelError("gemm: normed rows are not taken with this gated unit")
        pre = (scratch or _scratch_now(a.device))("gemm.glu_pre", (M, w.shape[0]), torch.float32)
        gemm(a, w, pre, EPI_STORE, force_generic, scratch)
        act_glu(pre, glu, c)
        return
    glu_args = glu.args(M) if glu is not None and not glu.plain else _NO_GLU
    act_args = _act_args(act, epilogue, "gemm")
    N = w.shape[0] // 2 if epilogue == EPI_SWIGLU else w.shape[0]   # swiglu: w holds gate rows, then up rows
    if w.shape[1] != K or tuple(c.shape) != (M, N):
        raise KernelError(f"gemm shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    if isinstance(a, NormedRows):
        if not gemm_can_norm_rows(M, w, c.dtype, epilogue):
            raise KernelError("gemm: normed rows are not taken for this product")
        _check(lib().llmx_gemm_skinny(0, _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), 0, 0, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, *a.args(), *act_args, *glu_args, _stream()),
               "gemm_skinny (normed rows)")
        return
    # a product wide enough to fill the chip with tiles (the LM head) streams its weights faster through the tiled kernel
    # from 5 rows on (every 16-feature strip of the weight-streaming kernel reads all rows again: 200,064 features at 8 rows
    # 264 against 239 us, at 16 rows 308 against 246 us); both kernels give a row the same bits
    skinny = M <= SKINNY_WIDE_MAX_ROWS or (M <= SKINNY_MAX_ROWS and -(-N // 128) < TILE_FILL)
    ks = _split_k(-(-N // 16), K)
    # some tens of rows: every 16-feature strip of the weight-streaming kernel reads all rows again; tiles of 128 features
    # do not, and are enough workgroups once each run of K has its own
    runs_apart = 0
    if scratch is not None and not force_generic and M >= TILE_RUNS_APART_MIN_ROWS and _skinny_ok(a, w, c, epilogue):
        runs_apart = lib().llmx_gemm_tile_runs_scratch(M, N, K, epilogue, ks, 0)
    if runs_apart:
        skinny = False
    if not force_generic and skinny and _skinny_ok(a, w, c, epilogue):
        _check(lib().llmx_gemm_skinny(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), 0, 0, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, *_NO_NORM, *act_args, *glu_args, _stream()),
               "gemm_skinny")
        return
    if not force_generic and _skinny_ok(a, w, c, epilogue):
        runs = scratch("gemm_tile.runs", (runs_apart,), torch.float32) if runs_apart else None
        _check(lib().llmx_gemm_tile(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), M, N, K, K, N, epilogue,
                                    ks, 0, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, 0, _dev(runs, "runs"), *act_args, *glu_args, _stream()), "gemm_tile")
        return
    _check(lib().llmx_gemm_generic(_dev(a, "a"), _code(a.dtype), _dev(w, "w"), _code(w.dtype), _dev(c, "c"), _code(c.dtype),
                                   M, N, K, K, K, N, epilogue, 0, 0, 0, 1, 0, N if epilogue == EPI_SWIGLU else 0, *act_args, *glu_args, _stream()), "gemm")


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor, a_div: int,
                 epilogue: int = EPI_STORE, active: Optional[torch.Tensor] = None, n_active: Optional[torch.Tensor] = None,
                 token_rows: Optional[int] = None, force_generic: bool = False, tile_stats: Optional[torch.Tensor] = None,
                 glu: Optional["Glu"] = None, scratch=None, act=None) -> None:
    """For each group g: rows p in pairs[offsets[g]:offsets[g+1]] get c[p] = a[p // a_div] @ w[g]^T.
    `act`: as gemm's, for the store epilogue.

    With EPI_SWIGLU w[g] holds gate rows then up rows and c[p] = silu(gate) * up.  `active` / `n_active` (from
    moe_align) list the groups that have rows; with them, steps of few token rows (`token_rows`, default the pair
    count) take the weight-streaming kernel.
    """
    G, NW, K = w.shape
    if _glu_apart(glu, epilogue):
        if isinstance(a, NormedRows):
            raise KernelError("grouped_gemm: normed rows are not taken with this gated unit")
        pre = (scratch or _scratch_now(a.device))("grouped_gemm.glu_pre", (c.shape[0], NW), torch.float32)
        grouped_gemm(a, w, pre, offsets, pairs, a_div, EPI_STORE, active, n_active, token_rows, force_generic, tile_stats)
        act_glu(pre, glu, c)
        return
    N = NW // 2 if epilogue == EPI_SWIGLU else NW
    if a.shape[1] != K or c.shape[1] != N:
        raise KernelError(f"grouped_gemm shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    n_pairs = pairs.shape[0]
    glu_args = glu.args(c.shape[0]) if glu is not None and not glu.plain else _NO_GLU
    act_args = _act_args(act, epilogue, "grouped_gemm")
    if c.shape[0] < n_pairs or a.shape[0] * a_div < n_pairs:
        raise KernelError("grouped_gemm: more pairs than rows")
    if token_rows is None:
        token_rows = n_pairs
    if isinstance(a, NormedRows):
        if active is None or n_active is None or act is not None or not gemm_can_norm_rows(a.shape[0], w, c.dtype, epilogue, grouped=True):
            raise KernelError("grouped_gemm: normed rows are not taken for this product")
        _check(lib().llmx_gemm_skinny(0, _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), G, min(G, n_pairs), _dev(active, "active", torch.int32, (G,)),
                                      _dev(n_active, "n_active", torch.int32, (1,)), _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                      _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, *a.args(), 0, 0, *glu_args, _stream()),
               "grouped_gemm_skinny (normed rows)")
        return
    if (not force_generic and active is not None and n_active is not None and _skinny_ok(a, w, c, epilogue)
            and token_rows <= SKINNY_MAX_GROUPED_ROWS):
        _check(lib().llmx_gemm_skinny(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                      _split_k(-(-N // 16), K), G, min(G, n_pairs), _dev(active, "active", torch.int32, (G,)),
                                      _dev(n_active, "n_active", torch.int32, (1,)), _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                      _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, *_NO_NORM, *act_args, *glu_args, _stream()),
               "grouped_gemm_skinny")
        return
    if not force_generic and _skinny_ok(a, w, c, epilogue):
        _check(lib().llmx_gemm_tile(_dev(a, "a"), _dev(w, "w"), _dev(c, "c"), _code(c.dtype), n_pairs, N, K, K, N, epilogue,
                                    _split_k(-(-N // 16), K), G, min(G, n_pairs) + n_pairs // 64, _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                    _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0,
                                    _dev(tile_stats if n_pairs >= TILE_STATS_MIN_PAIRS else None, "tile_stats", torch.int32, (1,)), 0, *act_args, *glu_args, _stream()),
               "grouped_gemm_tile")
        return
    _check(lib().llmx_gemm_generic(_dev(a, "a"), _code(a.dtype), _dev(w, "w"), _code(w.dtype), _dev(c, "c"), _code(c.dtype),
                                   n_pairs, N, K, K, K, N, epilogue, G, _dev(offsets, "offsets", torch.int32, (G + 1,)),
                                   _dev(pairs, "pairs", torch.int32), a_div, NW * K, N if epilogue == EPI_SWIGLU else 0, *act_args, *glu_args, _stream()),
           "grouped_gemm")


def qknorm_rope_kvwrite(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], cos_sin: torch.Tensor,
                        pos: torch.Tensor, row_entry: torch.Tensor, tables: torch.Tensor, q_out: torch.Tensor,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, eps: float, n_heads: int, n_kv_heads: int, head_dim: int,
                        rotary_dim: int, norm_mode: int, write_kv: bool = True, pairing: int = ROPE_HALVES) -> None:
    rows = qkv.shape[0]
    qw, kw = n_heads * head_dim, n_kv_heads * head_dim
    n_pages, hk, page_tokens, d = k_cache.shape
    if ((hk, d) != (n_kv_heads, head_dim) or tuple(v_cache.shape) != (n_pages, hk, d, page_tokens) or k_cache.dtype != q_out.dtype
            or v_cache.dtype != q_out.dtype):
        raise KernelError("qknorm_rope_kvwrite: cache shape or dtype does not fit the heads")
    if rotary_dim % 2 or rotary_dim > head_dim or cos_sin.shape[1] != rotary_dim:
        raise KernelError("qknorm_rope_kvwrite: rotary width does not fit")
    if norm_mode == QKNORM_PROJECTION:
        _dev(q_weight, "q_weight", torch.float32, (qw,))
        _dev(k_weight, "k_weight", torch.float32, (kw,))
    elif norm_mode != QKNORM_NONE:
        raise KernelError("qknorm_rope_kvwrite: only a norm over the whole projection, or none, is built")
    _check(lib().llmx_qknorm_rope_kvwrite(
        _dev(qkv, "qkv", torch.float32, (rows, qw + 2 * kw)), _dev(q_weight, "q_weight"), _dev(k_weight, "k_weight"),
        _dev(cos_sin, "cos_sin", torch.float32), _dev(pos, "pos", torch.int32, (rows,)), _dev(row_entry, "row_entry", torch.int32, (rows,)),
        _dev(tables, "tables", torch.int32), _dev(q_out, "q_out", shape=(rows, qw)), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _code(q_out.dtype), float(eps), rows, n_heads, n_kv_heads, head_dim, rotary_dim, norm_mode, page_tokens, tables.shape[1],
        1 if write_kv else 0, int(pairing), _stream()), "qknorm_rope_kvwrite")


def head_norm_rope_kvwrite(qkv: torch.Tensor, bias: Optional[torch.Tensor], q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                           cos_sin: torch.Tensor, pos: torch.Tensor, row_entry: torch.Tensor, tables: torch.Tensor, q_out: torch.Tensor,
                           k_cache: torch.Tensor, v_cache: torch.Tensor, eps: float, n_heads: int, n_kv_heads: int, head_dim: int,
                           rotary_dim: int, norm_mode: int, write_kv: bool = True, pairing: int = ROPE_HALVES,
                           q_scale: Optional[torch.Tensor] = None, maps: int = 1, values_from_keys: bool = False,
                           value_norm: bool = False) -> None:
    """qknorm_rope_kvwrite for heads that are treated one by one: float32 rows qkv = q (H*M*D) | k (G*M*D) | v (G*VD) get the
    projections' biases (`bias`, one vector of that width, or None), every q and k head an RMS norm over its own dims
    with a weight [D] shared by the heads (norm_mode QKNORM_HEAD; QKNORM_NONE: none), then the rotation; k and v go to the
    row's page.  The value width VD is the value cache's and may differ from D.  The rows may be wider than q | k | v (further
    columns of one fused projection follow v and are left alone).  `q_scale` [H*M] float32: the rotated q of head h is
    multiplied by q_scale[h] (a temperature a head on the scores, folded into the query).  `maps` M > 1: a head has M score
    maps, each with a query and a key head of its own ([head][map] in q's and k's columns and in the key cache) over one
    set of values.  `values_from_keys`: the rows hold no v; a value head is its key head as projected (before norm and
    rotation).  `value_norm`: a value head is divided by its root mean square (eps inside the root) before it is stored."""
    rows = qkv.shape[0]
    n_pages, hk, page_tokens, d = k_cache.shape
    v_dim = v_cache.shape[2]
    maps = int(maps)
    width = n_heads * maps * head_dim + n_kv_heads * maps * head_dim + (0 if values_from_keys else n_kv_heads * v_dim)
    if qkv.dim() != 2 or qkv.shape[1] < width:
        raise KernelError(f"head_norm_rope_kvwrite: rows of {tuple(qkv.shape)} do not hold q | k | v of {width} values")
    if ((hk, d) != (n_kv_heads * maps, head_dim) or tuple(v_cache.shape) != (n_pages, n_kv_heads, v_dim, page_tokens) or k_cache.dtype != q_out.dtype
            or v_cache.dtype != q_out.dtype):
        raise KernelError("head_norm_rope_kvwrite: cache shape or dtype does not fit the heads")
    if maps < 1 or (values_from_keys and (maps != 1 or v_dim != head_dim)):
        raise KernelError("head_norm_rope_kvwrite: values taken from the keys are as wide as they, one map a head")
    if rotary_dim % 2 or rotary_dim > head_dim or cos_sin.shape[1] != rotary_dim:
        raise KernelError("head_norm_rope_kvwrite: rotary width does not fit")
    if norm_mode not in (QKNORM_NONE, QKNORM_HEAD):
        raise KernelError("head_norm_rope_kvwrite: a norm a head, or none")
    if norm_mode == QKNORM_HEAD:
        _dev(q_weight, "q_weight", torch.float32, (head_dim,))
        _dev(k_weight, "k_weight", torch.float32, (head_dim,))
    _check(lib().llmx_head_norm_rope_kvwrite(
        _dev(qkv, "qkv", torch.float32), _dev(bias, "bias", torch.float32, (width,)), _dev(q_weight, "q_weight"),
        _dev(k_weight, "k_weight"), _dev(cos_sin, "cos_sin", torch.float32), _dev(pos, "pos", torch.int32, (rows,)),
        _dev(row_entry, "row_entry", torch.int32, (rows,)), _dev(tables, "tables", torch.int32),
        _dev(q_out, "q_out", shape=(rows, n_heads * maps * head_dim)),
        _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"), _code(q_out.dtype), float(eps), rows, n_heads * maps, n_kv_heads * maps, head_dim, v_dim,
        rotary_dim, norm_mode, page_tokens, tables.shape[1], 1 if write_kv else 0, int(pairing),
        _dev(q_scale, "q_scale", torch.float32, (n_heads * maps,)), qkv.shape[1], n_kv_heads, 1 if values_from_keys else 0,
        1 if value_norm else 0, _stream()), "head_norm_rope_kvwrite")


def gate_heads(o: torch.Tensor, gate: torch.Tensor, heads: int) -> None:
    """o[t, h*V + d] *= sigmoid(gate[t, h]), in place; o [T, heads * V] in its own type, gate a float32 view [T, heads] whose
    rows may be columns of a wider projection."""
    rows, width = o.shape
    if width % heads:
        raise KernelError(f"gate_heads: rows of {width} values are not {heads} heads")
    at, ldg = _rows_view(gate, "gate", rows, heads)
    _check(lib().llmx_gate_heads(_dev(o, "o"), _code(o.dtype), at, ldg, rows, heads, width // heads, _stream()), "gate_heads")


class AttentionPlan:
    """Work items of the matrix-core attention kernel for one step's rows (they hold no positions, so a plan serves
    every step with the same rows per request) and the merge list of the items that were split over the context."""

    def __init__(self, shared, items, merges, n_slots, device, merge_slots=0):
        import numpy as np
        self.n_shared = len(shared)          # prompt tiles, 12 (or three times 4) to a workgroup that shares their keys
        self.n_direct = sum(1 for i in items if i[6] < 0)
        items = shared + [i for i in items if i[6] < 0] + [i for i in items if i[6] >= 0]   # those that fold their segments first
        self.n_items = len(items)
        self.n_merges = len(merges)
        self.n_slots = n_slots
        # few decoding items: each is worked on by a workgroup of 4 waves (the kernel takes this form for head_dim 128)
        self.wide_items = 0 < self.n_items - self.n_shared <= ATTENTION_WIDE_ITEMS
        # no merged column longer than the merge's first loads reach
        self.short_merge = 0 < merge_slots <= lib().llmx_attention_partial_pad()
        self.items = torch.tensor(np.asarray(items, dtype=np.int32).reshape(-1, 8), device=device) if items else None
        self.merges = torch.tensor(np.asarray(merges, dtype=np.int32).reshape(-1, 8), device=device) if merges else None


_PLAN_CACHE: dict = {}
ATTENTION_TARGET_WAVES = 2048   # work items wanted before long contexts stop being split further
ATTENTION_WHOLE_ITEMS = 320     # from this many items on (rows x KV heads) no context is split: one wave an item walks its context (up to 512 items a workgroup each, over all the chip) at 5-6 TB/s, and sharing out would cost the partial results and their merge (4,096 tokens: 40 rows 163 -> 152 us a layer, 48 rows 190 -> 154, 64 rows 227 -> 176, 128 rows 447 -> 348; 32 rows are faster split: 114 against 139)
ATTENTION_SEGMENT = 128         # keys in a segment: the unit contexts are split in (the kernel's AM_SEG)
ATTENTION_WIDE_ITEMS = 1024     # up to this many decoding items a step, an item gets a workgroup of 4 waves instead of one wave


def attention_plan(row_counts, contexts, n_heads: int, n_kv_heads: int, device, window: int = 0) -> AttentionPlan:
    """row_counts[i]: rows of entry i in the step (entries' rows are consecutive, in order); contexts[i]: tokens the
    entry holds after the step.  Single-row entries become items per KV head (columns = its query heads) that share out
    the context's 128-key segments when there are few rows; longer entries become tiles of 16 rows of one head, 12 tiles
    that read the same KV head to a workgroup (three workgroups of 4 for head sizes other than 128).  How the context is shared out changes no result: segments are folded in
    key order either way."""
    ratio = n_heads // n_kv_heads
    head_chunks = [(kvh * ratio + c0, min(16, ratio - c0)) for kvh in range(n_kv_heads) for c0 in range(0, ratio, 16)]
    single = [i for i, n in enumerate(row_counts) if n == 1]
    n_splits, seg_cap = 1, 1
    if single:
        base = len(single) * len(head_chunks)
        longest = max(contexts[i] for i in single)
        if window > 0:
            longest = min(longest, window + ATTENTION_SEGMENT)
        seg_cap = -(-longest // ATTENTION_SEGMENT) + 1
        seg_cap = -(-seg_cap // 8) * 8       # in steps of 8, so a growing context reuses a plan for 1,024 tokens
        n_splits = max(1, min(-(-ATTENTION_TARGET_WAVES // base), seg_cap))
        if base >= ATTENTION_WHOLE_ITEMS:     # enough items as they are: sharing out would cost the partial results and their merge
            n_splits = 1
    key = (tuple(row_counts), n_heads, n_kv_heads, n_splits, seg_cap, str(device))
    plan = _PLAN_CACHE.get(key)
    if plan is not None:
        return plan
    shared, items, merges, slot = [], [], [], 0
    row0s, at = [], 0
    for n in row_counts:
        row0s.append(at)
        at += n
    # tiles of long entries, latest rows (longest key ranges) first; a KV head's last workgroup is filled up with empty items
    for i, n in enumerate(row_counts):
        if n == 1:
            continue
        per_head = []
        for kvh in range(n_kv_heads):
            tiles = [[row0s[i] + r0, min(16, n - r0), h, 1, 0, 1, -1, 0]
                     for r0 in range(((n - 1) // 16) * 16, -1, -16) for h in range(kvh * ratio, (kvh + 1) * ratio)]
            tiles += [[0, 0, 0, 1, 0, 1, -1, 0]] * (-len(tiles) % 12)
            per_head.append(tiles)
        for b in range(0, len(per_head[0]), 12):     # the KV heads' workgroups take turns, so long ranges start first
            for tiles in per_head:
                shared += tiles[b:b + 12]
    for i in single:
        for head0, nh in head_chunks:
            if n_splits == 1:
                items.append([row0s[i], 1, head0, nh, 0, 1, -1, 0])
                continue
            for c in range(nh):
                merges.append([row0s[i], head0 + c, slot, c, seg_cap, 0, 0, 0])
            for sp in range(n_splits):
                items.append([row0s[i], 1, head0, nh, sp, n_splits, slot, seg_cap])
            slot += seg_cap
    plan = AttentionPlan(shared, items, merges, slot, device, seg_cap)
    if len(_PLAN_CACHE) > 256:
        _PLAN_CACHE.clear()
    _PLAN_CACHE[key] = plan
    return plan


def attention_mfma_ok(dtype: torch.dtype, head_dim: int, page_tokens: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256 and page_tokens % 16 == 0


class ScoreRules:
    """What the universal attention kernel does to a row's scores and which keys it sees, beyond the causal rule and a
    window: keep_first (with a window: the request's first keys stay visible, at their true positions), chunk (a row sees
    only the keys of its own chunk of positions, counted from the request's start), softcap (score <- softcap tanh(score /
    softcap)), slopes (float32 [heads]: slopes[h] * (row's position - key's position) is taken off the score), sink (float32
    [heads]: one more logit a head in the softmax's denominator, without a key or a value), maps (score maps a head over one
    set of values: q [rows, heads * maps * head_dim], key cache of kv_heads * maps heads, out [rows, heads * maps * v_dim])."""

    def __init__(self, keep_first: int = 0, chunk: int = 0, softcap: float = 0.0, slopes: Optional[torch.Tensor] = None,
                 sink: Optional[torch.Tensor] = None, maps: int = 1):
        self.keep_first, self.chunk, self.softcap, self.slopes, self.sink, self.maps = int(keep_first), int(chunk), float(softcap), slopes, sink, int(maps)
        if self.keep_first < 0 or self.chunk < 0 or self.softcap < 0.0 or self.maps < 1 or (self.keep_first and self.chunk):
            raise KernelError("attention: keep_first, chunk and softcap are not negative, maps at least 1, and chunks keep no first keys")

    @property
    def plain(self) -> bool:
        return not (self.keep_first or self.chunk or self.softcap or self.slopes is not None or self.sink is not None or self.maps != 1)


class RulesPlan:
    """Work items of the matrix-core kernel that carries out ScoreRules (csrc/attention_rules.hip) for one step's rows; they
    hold no positions.  A tile's 16 columns are `hpc` query heads for each of 16 / hpc consecutive rows of one request.
    items [n, 8] int32: first row, rows, first head, this item's share and the number of shares its columns' segments are dealt
    into, first slot of the segments' partial sums (-1: the item folds its segments itself and stores the result), map;
    merges [n, 4]: row, head * maps + map, the column's first slot, slots from one segment to the next."""

    def __init__(self, items, merges, n_slots, hpc, device, group_items=()):
        import numpy as np
        self.n_items, self.n_merges, self.n_slots, self.hpc = len(items), len(merges), n_slots, hpc
        self.n_group_items = len(group_items)       # workgroups of four tiles of consecutive rows (prompt portions)
        self.group_items = torch.tensor(np.asarray(group_items, dtype=np.int32).reshape(-1, 8), device=device) if group_items else None
        self.items = torch.tensor(np.asarray(items, dtype=np.int32).reshape(-1, 8), device=device) if items else None
        self.merges = torch.tensor(np.asarray(merges, dtype=np.int32).reshape(-1, 4), device=device) if merges else None


RULES_SEGMENT = 128          # keys in a segment of the rules kernel (its AR_SEG)
RULES_CONTEXT_STEP = 1024    # a decoded row's context is rounded up to this for its plan, so that a growing context keeps its plan (and its graph) for long
_RULES_PLANS: dict = {}


def attention_rules_ok(dtype: torch.dtype, head_dim: int, v_dim: int, page_tokens: int) -> bool:
    return dtype == torch.bfloat16 and bool(lib().llmx_attention_rules_ok(BF16, int(head_dim), int(v_dim), int(page_tokens)))


def attention_rules_shared_ok(head_dim: int, v_dim: int) -> bool:
    """Whether the rules kernel has its four-wave form (keys and values through LDS) for these head widths."""
    return bool(lib().llmx_attention_rules_shared_ok(int(head_dim), int(v_dim)))


def rules_plan(row_counts, contexts, n_heads: int, n_kv_heads: int, maps: int, device, window: int = 0, keep_first: int = 0,
               chunk: int = 0, shared: bool = False) -> RulesPlan:
    """row_counts[i]: rows of entry i in the step (entries' rows are consecutive, in order); contexts[i]: tokens the entry
    holds after the step.  A tile takes the query heads of one key/value head together (where their number divides 16) for
    as many consecutive rows as 16 columns hold; a single-row entry (a decoded token) has its context's segments dealt into
    shares when the step has few rows.  How the context is shared out changes no result: segments are folded in key order
    either way.  `shared`: entries of several rows go to workgroups of four tiles that bring their keys and values from
    memory once (`attention_rules_shared_ok` says whether the kernel has that form for the head widths); the same bits."""
    if lib().llmx_attention_rules_segment() != RULES_SEGMENT:
        raise KernelError("rules_plan: the kernel library's segments are not the plan's")
    share = n_heads // n_kv_heads
    hpc = share if share <= 16 and 16 % share == 0 else 1
    groups = [(h0, m) for h0 in range(0, n_heads, hpc) for m in range(maps)]
    tile_rows = 16 // hpc
    rounded = tuple(-(-contexts[i] // RULES_CONTEXT_STEP) * RULES_CONTEXT_STEP if row_counts[i] == 1 else 0 for i in range(len(row_counts)))
    key = (tuple(row_counts), rounded, n_heads, n_kv_heads, maps, str(device), window, keep_first, chunk, bool(shared))
    hit = _RULES_PLANS.get(key)
    if hit is not None:
        return hit

    def segments_at_most(context):
        whole = -(-context // RULES_SEGMENT)
        if window > 0:
            whole = min(whole, -(-keep_first // RULES_SEGMENT) + window // RULES_SEGMENT + 2)
        if chunk > 0:
            whole = min(whole, chunk // RULES_SEGMENT + 2)
        return max(1, whole)

    single = [i for i, n in enumerate(row_counts) if n == 1]
    n_splits = {}
    if single:
        base = len(single) * len(groups)
        for i in single:
            n_splits[i] = max(1, min(segments_at_most(rounded[i]), ATTENTION_TARGET_WAVES // base))
    items, merges, group_items, slots, row = [], [], [], 0, 0
    for i, n in enumerate(row_counts):
        if n > 1 and shared:
            for r0 in reversed(range(0, n, 4 * tile_rows)):   # the longest contexts first
                for h0, m in groups:
                    group_items.append([row + r0, min(4 * tile_rows, n - r0), h0, 0, 1, -1, m, 0])
        elif n == 1 and n_splits[i] > 1:
            cap = segments_at_most(rounded[i])
            for h0, m in groups:
                for s in range(n_splits[i]):
                    items.append([row, 1, h0, s, n_splits[i], slots, m, 0])
                for c in range(hpc):
                    merges.append([row, (h0 + c) * maps + m, slots + c, hpc])
                slots += cap * hpc
        else:
            for r0 in reversed(range(0, n, tile_rows)):       # the tiles with the longest contexts first: they finish last otherwise
                for h0, m in groups:
                    items.append([row + r0, min(tile_rows, n - r0), h0, 0, 1, -1, m, 0])
        row += n
    plan = RulesPlan(items, merges, slots, hpc, device, group_items)
    if len(_RULES_PLANS) > 256:
        _RULES_PLANS.clear()
    _RULES_PLANS[key] = plan
    return plan


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: torch.Tensor, row_entry: torch.Tensor,
                    tables: torch.Tensor, out: torch.Tensor, scale: float, n_heads: int, window: int = 0,
                    plan: Optional[AttentionPlan] = None, scratch=None, head_gate: Optional[torch.Tensor] = None,
                    rules: Optional[ScoreRules] = None, output_gate: Optional[torch.Tensor] = None,
                    rules_plan: Optional[RulesPlan] = None) -> None:
    """Causal attention of each row over its request's pages.  With a `plan` (and bfloat16, head_dim a multiple of 16,
    pages of a multiple of 16 tokens, values as wide as keys) the matrix-core kernel runs; `scratch(name, shape, dtype)`
    gives it storage for the partial results of split contexts.  Otherwise the universal kernel runs; it takes values of
    a width of their own (v_cache [pages, kv_heads, v_dim, page_tokens], out [rows, heads * v_dim]).  `head_gate`: a float32
    view [rows, heads] (its rows may be columns of a wider projection): the result of (row, head) is multiplied by the
    sigmoid of its entry before it is stored, by whichever kernel stores it.  `output_gate`: such a view [rows, heads * v_dim],
    a logit a value of the result (the universal kernel).  `rules` (ScoreRules): the universal kernel's further score and
    visibility rules; with several maps `out` may be float32 whatever the cache's type (a later kernel joins the maps).
    `rules_plan` (from `rules_plan`, for this step's rows and these rules): where the sizes allow (`attention_rules_ok`) the
    matrix-core kernel for rules runs instead of the universal one."""
    rows = q.shape[0]
    maps = rules.maps if rules is not None else 1
    n_pages, key_heads, page_tokens, head_dim = k_cache.shape
    n_kv_heads = v_cache.shape[1]
    v_dim = v_cache.shape[2]
    if (q.shape[1] != n_heads * maps * head_dim or tuple(out.shape) != (rows, n_heads * maps * v_dim) or q.dtype != k_cache.dtype
            or (out.dtype != q.dtype and not (maps > 1 and out.dtype == torch.float32)) or v_cache.dtype != q.dtype or key_heads != n_kv_heads * maps):
        raise KernelError("paged_attention: shapes or dtypes do not agree")
    if head_dim > MAX_HEAD_DIM or v_dim > MAX_HEAD_DIM or n_heads % n_kv_heads:
        raise KernelError(f"paged_attention: head_dim {head_dim} or value width {v_dim} above {MAX_HEAD_DIM}, or heads {n_heads} not a multiple of KV heads {n_kv_heads}")
    common = (_dev(q, "q"), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache", shape=(n_pages, n_kv_heads, v_dim, page_tokens)),
              _dev(pos, "pos", torch.int32, (rows,)), _dev(row_entry, "row_entry", torch.int32, (rows,)), _dev(tables, "tables", torch.int32))
    gate_at, gate_ld = _rows_view(head_gate, "head_gate", rows, n_heads) if head_gate is not None else (None, 0)
    special = (rules is not None and not rules.plain) or output_gate is not None
    if plan is not None and plan.n_items and v_dim == head_dim and attention_mfma_ok(q.dtype, head_dim, page_tokens) and not special:
        part_o = part_ml = None
        if plan.n_slots:
            if scratch is None:
                scratch = lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=q.device)
            # the merge's loads run a fixed number of segments past a row's last one (never used)
            part_o = scratch("attention.part_o", (plan.n_slots * 16 + lib().llmx_attention_partial_pad(), head_dim), torch.float32)
            part_ml = scratch("attention.part_ml", (plan.n_slots * 16, 2), torch.float32)
        _check(lib().llmx_paged_attention_mfma(*common, _dev(plan.items, "items", torch.int32), plan.n_shared, plan.n_direct,
                                               plan.n_items - plan.n_shared - plan.n_direct,
                                               _dev(plan.merges, "merges", torch.int32), plan.n_merges, _dev(out, "out"),
                                               _dev(part_o, "part_o"), _dev(part_ml, "part_ml"), float(scale), n_heads, n_kv_heads,
                                               head_dim, page_tokens, tables.shape[1], int(window), (1 if plan.wide_items else 0) | (2 if plan.short_merge else 0), gate_at, gate_ld,
                                               _stream()),
               "paged_attention_mfma")
        return
    gate_wide = 0
    if output_gate is not None:
        if head_gate is not None or maps != 1:
            raise KernelError("paged_attention: one gate, and on one map a head")
        gate_at, gate_ld = _rows_view(output_gate, "output_gate", rows, n_heads * v_dim)
        gate_wide = 1
    r = rules if rules is not None else ScoreRules()
    if rules_plan is not None and (rules_plan.n_items or rules_plan.n_group_items) and attention_rules_ok(q.dtype, head_dim, v_dim, page_tokens):
        part_o = part_ml = None
        if rules_plan.n_slots:
            if scratch is None:
                scratch = lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device=q.device)
            part_o = scratch("attention.rules_part_o", (rules_plan.n_slots, v_dim), torch.float32)
            part_ml = scratch("attention.rules_part_ml", (rules_plan.n_slots, 2), torch.float32)
        _check(lib().llmx_attention_rules(*common, _dev(rules_plan.items, "items", torch.int32), rules_plan.n_items,
                                          _dev(rules_plan.group_items, "group_items", torch.int32), rules_plan.n_group_items,
                                          _dev(rules_plan.merges, "merges", torch.int32), rules_plan.n_merges, _dev(out, "out"),
                                          1 if out.dtype == torch.float32 else 0, _dev(part_o, "part_o"), _dev(part_ml, "part_ml"), float(scale),
                                          r.softcap, n_heads, n_kv_heads, r.maps, head_dim, v_dim, page_tokens, tables.shape[1], int(window),
                                          r.keep_first, r.chunk, _dev(r.slopes, "slopes", torch.float32, (n_heads,)),
                                          _dev(r.sink, "sink", torch.float32, (n_heads,)), gate_at, gate_ld, gate_wide, rules_plan.hpc, _stream()),
               "attention_rules")
        return
    _check(lib().llmx_paged_attention_generic(*common, _dev(out, "out"), _code(q.dtype), float(scale), rows, n_heads, n_kv_heads,
                                              head_dim, page_tokens, tables.shape[1], int(window), v_dim, gate_at, gate_ld, gate_wide,
                                              r.keep_first, r.chunk, r.maps, r.softcap, _dev(r.slopes, "slopes", torch.float32, (n_heads,)),
                                              _dev(r.sink, "sink", torch.float32, (n_heads,)), _code(out.dtype), _stream()), "paged_attention")


def _parts_args(z: torch.Tensor, parts: Optional[torch.Tensor]):
    if parts is None:
        return None, 1, 0
    if parts.dim() != 3 or tuple(parts.shape[1:]) != tuple(z.shape):
        raise KernelError(f"router partial sums {tuple(parts.shape)} do not fit logits {tuple(z.shape)}")
    return _dev(parts, "parts", torch.float32), parts.shape[0], z.numel()


def route_topk(z: torch.Tensor, bias: Optional[torch.Tensor], ids: torch.Tensor, weights: torch.Tensor, k: int, score: int,
               normalize: bool, scale: float, parts: Optional[torch.Tensor] = None, logit_bias: Optional[torch.Tensor] = None) -> None:
    """`parts` [slices, rows, experts]: the logits arrive as partial sums (gemm_f32's `parts`); they are added in slice
    order into z first.  `logit_bias` [experts]: added to the logits (z keeps the sum) before scores are formed.
    `normalize`: False, True (the picks' weights are divided by their sum; a single softmax pick keeps its score), or
    "always" (a single softmax pick is divided too: the softmax over the picked logits alone)."""
    rows, n_experts = z.shape
    if n_experts > MAX_EXPERTS or k > MAX_TOP_K or k > n_experts:
        raise KernelError(f"route_topk takes at most {MAX_EXPERTS} experts and {MAX_TOP_K} picks, not {n_experts} and {k}")
    _check(lib().llmx_route_topk(_dev(z, "z", torch.float32), *_parts_args(z, parts), _dev(bias, "bias", torch.float32, (n_experts,)),
                                 _dev(ids, "ids", torch.int32, (rows, k)), _dev(weights, "weights", torch.float32, (rows, k)),
                                 rows, n_experts, k, score, 2 if normalize == "always" else 1 if normalize else 0, float(scale),
                                 _dev(logit_bias, "logit_bias", torch.float32, (n_experts,)), _stream()), "route_topk")


def moe_align_scratch(n_pairs: int, n_experts: int) -> int:
    """Ints of scratch that moe_align wants for this many pairs (0: none)."""
    return 0 if n_pairs <= 1024 or n_experts > 1024 else -(-n_pairs // 1024) * n_experts


TILE_STATS_MIN_PAIRS = 4096    # from this many pairs on the grouping also counts the experts' tiles of 128 rows


def moe_align(ids: torch.Tensor, n_experts: int, counts: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor,
              active: torch.Tensor, n_active: torch.Tensor, scratch: Optional[torch.Tensor] = None,
              tile_stats: Optional[torch.Tensor] = None) -> None:
    """Groups the pairs p = t*k + j by expert (stable): counts [X], offsets [X+1], pairs [T*k], and the experts that
    have rows in increasing order: active [X] (first n_active[0] entries).  `scratch`: moe_align_scratch(...) int32 for
    steps of many pairs (made here when it is not given).  `tile_stats` int32 [1]: for TILE_STATS_MIN_PAIRS pairs or
    more it receives the sum over experts of ceil(rows / 128), by which grouped_gemm chooses its tile size."""
    n_pairs = ids.numel()
    need = moe_align_scratch(n_pairs, n_experts)
    if need and scratch is None:
        scratch = torch.empty(need, dtype=torch.int32, device=ids.device)
    if scratch is not None and scratch.numel() < need:
        raise KernelError(f"moe_align: scratch of {scratch.numel()} ints, {need} needed")
    _check(lib().llmx_moe_align(_dev(ids, "ids", torch.int32), n_pairs, n_experts, _dev(counts, "counts", torch.int32, (n_experts,)),
                                _dev(offsets, "offsets", torch.int32, (n_experts + 1,)), _dev(pairs, "pairs", torch.int32, (n_pairs,)),
                                _dev(active, "active", torch.int32, (n_experts,)), _dev(n_active, "n_active", torch.int32, (1,)),
                                _dev(scratch if need else None, "scratch", torch.int32),
                                _dev(tile_stats if need and n_pairs >= TILE_STATS_MIN_PAIRS else None, "tile_stats", torch.int32, (1,)),
                                _stream()), "moe_align")


def route_topk_align(z: torch.Tensor, bias: Optional[torch.Tensor], ids: torch.Tensor, weights: torch.Tensor, k: int, score: int,
                     normalize: bool, scale: float, counts: torch.Tensor, offsets: torch.Tensor, pairs: torch.Tensor,
                     active: torch.Tensor, n_active: torch.Tensor, parts: Optional[torch.Tensor] = None,
                     scratch: Optional[torch.Tensor] = None, tile_stats: Optional[torch.Tensor] = None,
                     logit_bias: Optional[torch.Tensor] = None) -> None:
    """route_topk followed by moe_align; a step of at most 16 rows (sigmoid scores, at most 256 experts and 64 picks) does
    both in one launch, with the same bits."""
    rows, n_experts = z.shape
    if score == SCORE_SIGMOID and rows <= 16 and rows * k <= 1024 and n_experts <= 256 and k <= 64 and logit_bias is None and normalize != "always":
        _check(lib().llmx_route_topk_align(
            _dev(z, "z", torch.float32), *_parts_args(z, parts), _dev(bias, "bias", torch.float32, (n_experts,)),
            _dev(ids, "ids", torch.int32, (rows, k)),
            _dev(weights, "weights", torch.float32, (rows, k)), rows, n_experts, k, 1 if normalize else 0, float(scale),
            _dev(counts, "counts", torch.int32, (n_experts,)), _dev(offsets, "offsets", torch.int32, (n_experts + 1,)),
            _dev(pairs, "pairs", torch.int32, (rows * k,)), _dev(active, "active", torch.int32, (n_experts,)),
            _dev(n_active, "n_active", torch.int32, (1,)), _stream()), "route_topk_align")
        return
    route_topk(z, bias, ids, weights, k, score, normalize, scale, parts, logit_bias)
    moe_align(ids, n_experts, counts, offsets, pairs, active, n_active, scratch, tile_stats)


def moe_combine(x: torch.Tensor, y: torch.Tensor, ids: torch.Tensor, weights: Optional[torch.Tensor], accumulate: bool = True) -> None:
    """x[t] (+)= sum over the row's slots j of weights[t, j] * y[t*k + j] in slot order (weights None: every weight 1)."""
    rows, width = x.shape
    k = ids.shape[1]
    _check(lib().llmx_moe_combine(_dev(x, "x", torch.float32), _dev(y, "y", torch.float32, (rows * k, width)),
                                  _dev(ids, "ids", torch.int32, (rows, k)), _dev(weights, "weights", torch.float32, (rows, k)),
                                  rows, k, width, 1 if accumulate else 0, _stream()), "moe_combine")


def fill_i32(t: torch.Tensor, value: int) -> None:
    _check(lib().llmx_fill_i32(_dev(t, "t", torch.int32), int(value), t.numel(), _stream()), "fill_i32")


def fill_random(t: torch.Tensor, key: int, kind: int, a: float, b: float) -> None:
    """Seeded fill: kind 0 = a + b * normal, kind 1 = uniform in [a, b); element i depends on (key, i) only."""
    _check(lib().llmx_fill_random(_dev(t, "t"), _code(t.dtype), t.numel(), key & ((1 << 64) - 1), int(kind), float(a), float(b),
                                  _stream()), "fill_random")


def read_probe(t: torch.Tensor, out: torch.Tensor) -> None:
    """Streams the tensor's bytes (a multiple of 16) through a kernel that keeps nothing: a measure of the card's read rate."""
    _check(lib().llmx_read_probe(_dev(t, "t"), t.numel() * t.element_size(), _dev(out, "out", torch.int32), _stream()), "read_probe")


_SCRATCH: dict = {}


def _scratch(name: str, count: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A cached device buffer of at least `count` elements (grown, never shrunk): storage the kernels need besides their operands."""
    key = (name, dtype, str(device))
    t = _SCRATCH.get(key)
    if t is None or t.numel() < count:
        t = torch.empty(max(count, 1), dtype=dtype, device=device)
        _SCRATCH[key] = t
    return t


def argmax_rows(scores: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None) -> None:
    rows, n = scores.shape
    partial = _scratch("argmax.partial", 2 * rows * (-(-n // 8192)), torch.int32, scores.device) if n > 16384 else None
    _check(lib().llmx_argmax_rows(_dev(scores, "scores", torch.float32), _dev(skip, "skip", torch.int32, (rows,)),
                                  _dev(out, "out", torch.int32, (rows,)), _dev(partial, "partial"), rows, n, _stream()), "argmax_rows")


def gemm_f32_slices(N: int, K: int) -> int:
    """Runs that gemm_f32 cuts K into when its caller takes partial sums (a function of the weight's shape only)."""
    if K % 4:
        return 1
    n_strips, steps, s = -(-N // 16), K // 16, 1
    while s < 8 and n_strips * s < 128 and steps // (s * 2) >= 12:
        s *= 2
    return s


def gemm_f32(a, w: torch.Tensor, c: torch.Tensor, add: bool = False, parts: Optional[torch.Tensor] = None) -> None:
    """c[M,N] (+)= a[M,K] @ w[N,K]^T, everything float32, on the float32 matrix instruction (the router's product).
    A row's bits depend on the shape of w only.  K a multiple of 4; otherwise the universal kernel runs.
    `parts` [gemm_f32_slices(N, K), M, N] with more than one slice: K's runs are written there instead of c, spread over
    that many more workgroups, and the reader (route_topk) adds them in order."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(c.shape) != (M, N):
        raise KernelError(f"gemm_f32 shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    normed = isinstance(a, NormedRows)    # the product reads norm(x), unrounded, formed by its own workgroups
    if normed and not gemm_f32_can_norm_rows(M, w):
        raise KernelError("gemm_f32: normed rows are not taken for this product")
    if K % 4:
        if parts is not None:
            raise KernelError("gemm_f32: partial sums need K to be a multiple of 4")
        gemm(a, w, c, EPI_ADD if add else EPI_STORE, force_generic=True)
        return
    slices = 1
    if parts is not None:
        slices = parts.shape[0]
        if tuple(parts.shape) != (gemm_f32_slices(N, K), M, N) or add:
            raise KernelError(f"gemm_f32: partial sums {tuple(parts.shape)} for {(M, N)} with add={add}")
    ks = 1
    n_strips = -(-N // 16)
    steps = (K // 16) // slices
    while ks < 16 and n_strips * slices * ks < 1024 and steps // (ks * 2) >= (8 if slices == 1 else 3):   # from w's shape only
        ks *= 2
    target = parts if parts is not None else c
    _check(lib().llmx_gemm_skinny_f32(_dev(a.x if normed else a, "a", torch.float32), _dev(w, "w", torch.float32), _dev(target, "c", torch.float32),
                                      M, N, K, K, N, 1 if add else 0, ks, slices, M * N,
                                      _dev(a.weight, "norm weight", torch.float32, (K,)) if normed else 0, a.eps if normed else 0.0, _stream()),
           "gemm_f32")


def sample_all(scores: torch.Tensor, temp: torch.Tensor, unit: torch.Tensor, out: torch.Tensor, min_p: Optional[torch.Tensor] = None,
               skip: Optional[torch.Tensor] = None, slices: bool = True) -> None:
    """The temperature draw with every token kept.  Rows of many scores are summed by many workgroups (a slice of 8,192
    scores each) and one more a row finds the token; `slices=False` keeps a row to one workgroup.  The orders of the
    double additions differ between the two, so their targets can differ in the last bits of a double."""
    rows, n = scores.shape
    need = lib().llmx_sample_all_scratch(rows, n) if slices else 0
    scratch = _scratch("sample_all.slices", -(-need // 8), torch.float64, scores.device) if need else None
    _check(lib().llmx_sample_all(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                 _dev(unit, "unit", torch.float32, (rows,)), _dev(min_p, "min_p", torch.float32, (rows,)),
                                 _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                 _dev(scratch, "scratch"), _stream()), "sample_all")


def sample_topk(scores: torch.Tensor, temp: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, min_p: torch.Tensor,
                unit: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None, max_keep: int = 1024, slices: bool = True) -> None:
    """Top-k (1..1024 per row), top-p, min-p and the draw; rows whose top_k is outside 1..1024 must not be read from `out`.
    `max_keep`: no row's top_k is above it (it sizes the scratch).  Rows of many scores are searched by many workgroups
    (each keeps the best of a slice, one more ranks the slices' candidates and draws); `slices=False` keeps a row to one
    workgroup.  The token is the same either way."""
    rows, n = scores.shape
    need = lib().llmx_sample_topk_scratch(rows, n, int(max_keep)) if slices else 0
    cand = _scratch("sample_topk.candidates", need, torch.int32, scores.device) if need else None
    _check(lib().llmx_sample_topk(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                  _dev(top_k, "top_k", torch.int32, (rows,)), _dev(top_p, "top_p", torch.float32, (rows,)),
                                  _dev(min_p, "min_p", torch.float32, (rows,)), _dev(unit, "unit", torch.float32, (rows,)),
                                  _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                  _dev(cand, "candidates"), int(max_keep), _stream()), "sample_topk")


def sample_ranked(scores: torch.Tensor, temp: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, min_p: torch.Tensor,
                  unit: torch.Tensor, out: torch.Tensor, skip: Optional[torch.Tensor] = None, slices: bool = True) -> Optional[torch.Tensor]:
    """Top-k of any size (0 keeps all), top-p, min-p and the draw, without sorting; rows with temp <= 0 are left unwritten.
    A nucleus over a whole row of many scores is looked for among the best 256 of every slice of 8,192 scores, which many
    workgroups find; a row whose nucleus is not certain to lie among them (or that has a top_k) is then walked whole by
    one workgroup, as every row is with `slices=False`.  The token is the same either way.  Returns, when the search by
    slices ran, a device tensor with 1 for every row that was walked whole after it (a view of scratch the next call
    overwrites), else None."""
    rows, n = scores.shape
    need = lib().llmx_sample_ranked_scratch(rows, n) if slices else 0
    scratch = _scratch("sample_ranked.slices", -(-need // 8), torch.float64, scores.device) if need else None
    _check(lib().llmx_sample_ranked(_dev(scores, "scores", torch.float32), _dev(temp, "temp", torch.float32, (rows,)),
                                    _dev(top_k, "top_k", torch.int32, (rows,)), _dev(top_p, "top_p", torch.float32, (rows,)),
                                    _dev(min_p, "min_p", torch.float32, (rows,)), _dev(unit, "unit", torch.float32, (rows,)),
                                    _dev(skip, "skip", torch.int32, (rows,)), _dev(out, "out", torch.int32, (rows,)), rows, n,
                                    _dev(scratch, "scratch"), _stream()), "sample_ranked")
    if scratch is None:
        return None
    return scratch.view(torch.int32)[need // 4 - rows:need // 4]


def penalize(scores: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor, penalty: torch.Tensor,
             presence: torch.Tensor, frequency: torch.Tensor) -> None:
    """In place: for each (rows[i], ids[i]) seen counts[i] times, the repetition, presence and frequency penalties."""
    W, n = scores.shape
    n_seen = rows.shape[0]
    _check(lib().llmx_penalize(_dev(scores, "scores", torch.float32), _dev(rows, "rows", torch.int32), _dev(ids, "ids", torch.int32, (n_seen,)),
                               _dev(counts, "counts", torch.int32, (n_seen,)), _dev(penalty, "penalty", torch.float32, (W,)),
                               _dev(presence, "presence", torch.float32, (W,)), _dev(frequency, "frequency", torch.float32, (W,)),
                               n_seen, n, _stream()), "penalize")
