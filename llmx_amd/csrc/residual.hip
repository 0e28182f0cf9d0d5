// Kernels around the residual stream of layers whose mixer and feed-forward read the same rows: one norm pass with two
// gains, the scaled join of both results, a normed join, and activations applied between two products.
// Everything here is float32 arithmetic on float32 rows; only what a product reads next is stored in the activation type.
#include "common.h"

// ---------------------------------------------------------------------------
// Two RMS norms of the same row with the same eps and different gains: r is formed once (the sum of squares in the
// order of rmsnorm_kernel, so each output has the bits that kernel gives with its gain), out1 = x * (r * w1),
// out2 = x * (r * w2).  out2 / w2 may be null.
#define PAIR_THREADS 1024
template <typename TO>
__global__ void __launch_bounds__(PAIR_THREADS) rmsnorm_pair_kernel(const float* __restrict__ x, const float* __restrict__ w1,
                                                                  const float* __restrict__ w2, float eps, TO* __restrict__ out1,
                                                                  TO* __restrict__ out2, int n) {
    __shared__ float scratch[PAIR_THREADS / 64];
    const int r = blockIdx.x;
    const float* row = x + (size_t)r * n;
    const float s = block_sum<PAIR_THREADS / 64>(strided_squares<PAIR_THREADS>(row, n), scratch);
    const float scale = 1.0f / sqrtf(s / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += PAIR_THREADS) {
        const float v = row[i];
        st(out1 + (size_t)r * n + i, v * (scale * w1[i]));
        if (out2) st(out2 + (size_t)r * n + i, v * (scale * w2[i]));
    }
}

extern "C" int llmx_rmsnorm_pair(const float* x, const float* w1, const float* w2, float eps, void* out1, void* out2, int out_dtype,
                                 int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (!w1 || !out1 || ((out2 != nullptr) != (w2 != nullptr))) return -2;
    llmx_note_launch(LK_RMSNORM_PAIR);
    if (out_dtype == LLMX_F32)
        hipLaunchKernelGGL(rmsnorm_pair_kernel<float>, dim3(rows), dim3(PAIR_THREADS), 0, stream, x, w1, w2, eps, (float*)out1, (float*)out2, n);
    else
        hipLaunchKernelGGL(rmsnorm_pair_kernel<bf16_t>, dim3(rows), dim3(PAIR_THREADS), 0, stream, x, w1, w2, eps, (bf16_t*)out1, (bf16_t*)out2, n);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// x[t,i] += s1[i] * y1[t,i] + s2[i] * y2[t,i] (the second term only when y2 is given; a null scale is 1), and
// optionally a copy of the new row in the activation type for the product that reads it next.
template <typename TO>
__global__ void __launch_bounds__(256) scale_add_kernel(float* __restrict__ x, const float* __restrict__ y1, const float* __restrict__ s1,
                                                      const float* __restrict__ y2, const float* __restrict__ s2, TO* __restrict__ copy,
                                                      int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    const int i = (int)(at % (size_t)n);
    float joined = y1[at] * (s1 ? s1[i] : 1.0f);
    if (y2) joined = joined + y2[at] * (s2 ? s2[i] : 1.0f);
    const float v = x[at] + joined;
    x[at] = v;
    if (copy) st(copy + at, v);
}

extern "C" int llmx_scale_add(float* x, const float* y1, const float* s1, const float* y2, const float* s2, void* copy, int copy_dtype,
                              int rows, int n, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    llmx_note_launch(LK_SCALE_ADD);
    const size_t total = (size_t)rows * n;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (copy_dtype == LLMX_F32)
        hipLaunchKernelGGL(scale_add_kernel<float>, grid, dim3(256), 0, stream, x, y1, s1, y2, s2, (float*)copy, n, total);
    else
        hipLaunchKernelGGL(scale_add_kernel<bf16_t>, grid, dim3(256), 0, stream, x, y1, s1, y2, s2, (bf16_t*)copy, n, total);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// x[t,:] += y[t,:] * (r * w[:]), r = 1 / sqrt(mean(y[t,:]^2) + eps): a result joined after its own RMS norm.  One block of
// 1,024 threads a row; the sum as the norm kernels form it (a thread's elements in stride order with fmaf, a butterfly a
// wave, the waves in order), which is also the first sum of rmsnorm_add_norm_kernel: both give x the same bits.  Rows of at
// most 8,192 values are kept in registers, all loads asked for before the sum.
#define ADD_THREADS 1024
#define ADD_KEPT 8
__global__ void __launch_bounds__(ADD_THREADS) rmsnorm_add_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w,
                                                                 float eps, int n) {
    __shared__ float scratch[ADD_THREADS / 64];
    const int r = blockIdx.x;
    const float* row = y + (size_t)r * n;
    float* out = x + (size_t)r * n;
    if (n <= ADD_THREADS * ADD_KEPT) {
        float vx[ADD_KEPT], vy[ADD_KEPT], wj[ADD_KEPT];
#pragma unroll
        for (int e = 0; e < ADD_KEPT; ++e) {
            const int i = threadIdx.x + e * ADD_THREADS;
            const bool in = i < n;
            vy[e] = in ? row[i] : 0.0f;
            vx[e] = in ? out[i] : 0.0f;
            wj[e] = in ? w[i] : 0.0f;
        }
        float sq = 0.0f;
#pragma unroll
        for (int e = 0; e < ADD_KEPT; ++e) sq = fmaf(vy[e], vy[e], sq);
        const float scale = 1.0f / sqrtf(block_sum<ADD_THREADS / 64>(sq, scratch) / (float)n + eps);
#pragma unroll
        for (int e = 0; e < ADD_KEPT; ++e) {
            const int i = threadIdx.x + e * ADD_THREADS;
            if (i < n) out[i] = vx[e] + vy[e] * (scale * wj[e]);
        }
        return;
    }
    float sq = 0.0f;
    for (int i = threadIdx.x; i < n; i += ADD_THREADS) sq = fmaf(row[i], row[i], sq);
    const float scale = 1.0f / sqrtf(block_sum<ADD_THREADS / 64>(sq, scratch) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += ADD_THREADS) out[i] = out[i] + row[i] * (scale * w[i]);
}

extern "C" int llmx_rmsnorm_add(float* x, const float* y, const float* w, float eps, int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    llmx_note_launch(LK_RMSNORM_ADD);
    hipLaunchKernelGGL(rmsnorm_add_kernel, dim3(rows), dim3(ADD_THREADS), 0, stream, x, y, w, eps, n);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// Activations between two products, float32 in, the activation type out.
// xIELU with the two numbers (p, q) of `pq`: z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2.
// Four neighbouring values a thread (one 16-byte load); the last thread takes what is left one by one.
template <typename TO>
__global__ void __launch_bounds__(256) xielu_kernel(const float* __restrict__ z, const float* __restrict__ pq, TO* __restrict__ out, size_t total) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const size_t at = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
    if (at >= total) return;
    const ActFn act(LLMX_ACT_XIELU, pq);
    if (at + 4 <= total) {
        const f32x4_t v = *reinterpret_cast<const f32x4_t*>(z + at);
#pragma unroll
        for (int i = 0; i < 4; ++i) st(out + at + i, act(v[i]));
        return;
    }
    for (size_t i = at; i < total; ++i) st(out + i, act(z[i]));
}

extern "C" int llmx_act_xielu(const float* z, const float* pq, void* out, int out_dtype, long total, hipStream_t stream) {
    if (total <= 0) return 0;
    llmx_note_launch(LK_ACT_XIELU);
    const dim3 grid((unsigned)((total + 1023) / 1024));
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(xielu_kernel<float>, grid, dim3(256), 0, stream, z, pq, (float*)out, (size_t)total);
    else hipLaunchKernelGGL(xielu_kernel<bf16_t>, grid, dim3(256), 0, stream, z, pq, (bf16_t*)out, (size_t)total);
    return LLMX_CHECK_LAUNCH();
}

// out[t,j] = gelu_tanh(z[t,j]) * table[ids[t], col0 + j], j < n: a gate on a slice of a token table's row.
// gelu_tanh(v) = v/2 (1 + tanh(sqrt(2/pi) (v + 0.044715 v^3))).
template <typename TT, typename TO>
__global__ void __launch_bounds__(256) gelu_gather_kernel(const float* __restrict__ z, const TT* __restrict__ table, const int* __restrict__ ids,
                                                        TO* __restrict__ out, int n, int col0, int table_ld, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    const int t = (int)(at / (size_t)n), j = (int)(at % (size_t)n);
    const float v = z[at];
    const float g = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    st(out + at, g * ld(table + (size_t)ids[t] * table_ld + col0 + j));
}

extern "C" int llmx_act_gelu_gather(const float* z, const void* table, int table_dtype, const int* ids, void* out, int out_dtype, int rows,
                                    int n, int col0, int table_ld, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    if (col0 < 0 || col0 + n > table_ld) return -2;
    llmx_note_launch(LK_ACT_GELU_GATHER);
    const size_t total = (size_t)rows * n;
    const dim3 grid((unsigned)((total + 255) / 256));
#define LLMX_GG(TT, TO) hipLaunchKernelGGL((gelu_gather_kernel<TT, TO>), grid, dim3(256), 0, stream, z, (const TT*)table, ids, (TO*)out, n, col0, table_ld, total)
    if (table_dtype == LLMX_F32 && out_dtype == LLMX_F32) LLMX_GG(float, float);
    else if (table_dtype == LLMX_F32) LLMX_GG(float, bf16_t);
    else if (out_dtype == LLMX_F32) LLMX_GG(bf16_t, float);
    else LLMX_GG(bf16_t, bf16_t);
#undef LLMX_GG
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// x[t,:] = (x[t,:] + rows[t,:]) + vec[:]: what a repeated run of layers adds to the residual before a pass (rows: a kept
// copy of earlier rows, or null; vec: the pass's own vector).
__global__ void __launch_bounds__(256) add_rows_vector_kernel(float* __restrict__ x, const float* __restrict__ rows, const float* __restrict__ vec,
                                                            int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    float v = x[at];
    if (rows) v = v + rows[at];
    if (vec) v = v + vec[(int)(at % (size_t)n)];
    x[at] = v;
}

extern "C" int llmx_add_rows_vector(float* x, const float* rows, const float* vec, int n_rows, int n, hipStream_t stream) {
    if (n_rows <= 0 || n <= 0) return 0;
    llmx_note_launch(LK_ADD_ROWS_VECTOR);
    const size_t total = (size_t)n_rows * n;
    hipLaunchKernelGGL(add_rows_vector_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, rows, vec, n, total);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// A polynomial of unit-RMS powers between two products: with U(v) = v / sqrt(mean(v^2) + eps) over a row,
// out = a U(z) + b U(z^2) + c U(z^3) + e, powers element by element, (a, b, c, e) four numbers on the device.  A block of
// 1,024 threads a row: the sums of z^2, z^4 and z^6 in one pass (a thread's elements in stride order with fmaf, then
// block_sum), then the row again.  Rows of at most 16,384 values stay in registers between the two passes, every load asked
// for before the first sum, so the kernel waits for memory once; longer rows are read again (they are still in the
// caches).  The same operations in the same order either way.  Everything float32; only the result is stored in the
// activation type.
#define POLY_THREADS 1024
#define POLY_KEPT 16
template <typename TO, int KEPT>
__global__ void __launch_bounds__(POLY_THREADS) polynorm_kernel(const float* __restrict__ z, const float* __restrict__ abce, float eps,
                                                              TO* __restrict__ out, int n) {
    __shared__ float scratch[POLY_THREADS / 64];
    const int r = blockIdx.x;
    const float* row = z + (size_t)r * n;
    const float a = abce[0], b = abce[1], c = abce[2], e = abce[3];
    float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
    auto add = [&](float v) {
        const float p2 = v * v, p3 = p2 * v;
        s2 = fmaf(v, v, s2);
        s4 = fmaf(p2, p2, s4);
        s6 = fmaf(p3, p3, s6);
    };
    auto factors = [&](float& r1, float& r2, float& r3) {
        s2 = block_sum<POLY_THREADS / 64>(s2, scratch);
        s4 = block_sum<POLY_THREADS / 64>(s4, scratch);
        s6 = block_sum<POLY_THREADS / 64>(s6, scratch);
        r1 = a / sqrtf(s2 / (float)n + eps);
        r2 = b / sqrtf(s4 / (float)n + eps);
        r3 = c / sqrtf(s6 / (float)n + eps);
    };
    auto value = [&](float v, float r1, float r2, float r3) {
        const float p2 = v * v;
        return ((v * r1 + p2 * r2) + (p2 * v) * r3) + e;
    };
    float r1, r2, r3;
    if (n <= POLY_THREADS * KEPT) {
        float v[KEPT];
#pragma unroll
        for (int u = 0; u < KEPT; ++u) {
            const int i = threadIdx.x + u * POLY_THREADS;
            v[u] = i < n ? row[i] : 0.0f;           // an element past the end adds fmaf(0, 0, s) = s
        }
#pragma unroll
        for (int u = 0; u < KEPT; ++u) add(v[u]);
        factors(r1, r2, r3);
#pragma unroll
        for (int u = 0; u < KEPT; ++u) {
            const int i = threadIdx.x + u * POLY_THREADS;
            if (i < n) st(out + (size_t)r * n + i, value(v[u], r1, r2, r3));
        }
        return;
    }
    for (int i = threadIdx.x; i < n; i += 4 * POLY_THREADS) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * POLY_THREADS < n ? row[i + u * POLY_THREADS] : 0.0f;
#pragma unroll
        for (int u = 0; u < 4; ++u) add(v[u]);
    }
    factors(r1, r2, r3);
    for (int i = threadIdx.x; i < n; i += POLY_THREADS) st(out + (size_t)r * n + i, value(row[i], r1, r2, r3));
}

extern "C" int llmx_act_polynorm(const float* z, const float* abce, float eps, void* out, int out_dtype, int rows, int n, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    llmx_note_launch(LK_ACT_POLYNORM);
    // half the registers where a row fits them: more rows on a compute unit at a time
#define POLY_LAUNCH(TO, KEPT) hipLaunchKernelGGL((polynorm_kernel<TO, KEPT>), dim3(rows), dim3(POLY_THREADS), 0, stream, z, abce, eps, (TO*)out, n)
    if (out_dtype == LLMX_F32) {
        if (n <= POLY_THREADS * POLY_KEPT / 2) POLY_LAUNCH(float, POLY_KEPT / 2);
        else POLY_LAUNCH(float, POLY_KEPT);
    } else {
        if (n <= POLY_THREADS * POLY_KEPT / 2) POLY_LAUNCH(bf16_t, POLY_KEPT / 2);
        else POLY_LAUNCH(bf16_t, POLY_KEPT);
    }
#undef POLY_LAUNCH
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// A gated unit between two products, as a kernel of its own (GluFn: silu(gate) * up, or the clamped form): a row of `pre`
// holds n gate values, then n up values (row stride ld); with s = row_scale[p] (a factor on the row's *input*, which the first
// product being linear is a factor on both pre-activations; null: 1): out = unit(s gate, s up), times
// sigmoid(row_gate[p * row_gate_ld]) where a gate logit a row is given.
template <typename TO>
__global__ void __launch_bounds__(256) glu_kernel(const float* __restrict__ pre, int ld, const float* __restrict__ row_scale,
                                                        const float* __restrict__ row_gate, int row_gate_ld, int kind, float limit, TO* __restrict__ out,
                                                        int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    const size_t p = at / (size_t)n;
    const int j = (int)(at % (size_t)n);
    const GluFn glu(kind, limit);
    const float s = row_scale ? row_scale[p] : 1.0f;
    float y = glu(pre[p * ld + j] * s, pre[p * ld + n + j] * s);
    if (row_gate) y = y * sigmoid_f(row_gate[p * row_gate_ld]);
    st(out + at, y);
}

extern "C" int llmx_act_glu(const float* pre, int ld, const float* row_scale, const float* row_gate, int row_gate_ld, int kind, float limit,
                            void* out, int out_dtype, int rows, int n, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    if (ld < 2 * n || (kind != LLMX_GLU_SILU && kind != LLMX_GLU_CLAMPED && kind != LLMX_GLU_GELU_TANH) || (kind == LLMX_GLU_CLAMPED && !(limit > 0.0f))) return -2;
    llmx_note_launch(LK_ACT_GLU);
    const size_t total = (size_t)rows * n;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (out_dtype == LLMX_F32)
        hipLaunchKernelGGL(glu_kernel<float>, grid, dim3(256), 0, stream, pre, ld, row_scale, row_gate, row_gate_ld, kind, limit, (float*)out, n, total);
    else
        hipLaunchKernelGGL(glu_kernel<bf16_t>, grid, dim3(256), 0, stream, pre, ld, row_scale, row_gate, row_gate_ld, kind, limit, (bf16_t*)out, n, total);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// A result joined after its own RMS norm, and the next sublayer's norm of the new row, in one pass:
// x[t,:] += y[t,:] * (r_y * w_join[:]); h[t,:] = x[t,:] * (r_x * w_next[:]), r_v = 1 / sqrt(mean(v^2) + eps_v).
// One block of 1,024 threads a row; rows of at most 8,192 values stay in registers between the two sums (every load is
// asked for before the first sum), longer rows are read again.  Each sum: a thread's elements in stride order with fmaf, a
// butterfly a wave, the waves in order.  h is stored in the activation type and/or as float32.
#define JOIN_THREADS 1024
#define JOIN_KEPT 8
template <typename TO>
__global__ void __launch_bounds__(JOIN_THREADS) rmsnorm_add_norm_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                      const float* __restrict__ w_join, float eps_join,
                                                                      const float* __restrict__ w_next, float eps_next, TO* __restrict__ out,
                                                                      float* __restrict__ out32, int n) {
    __shared__ float scratch[JOIN_THREADS / 64];
    const int r = blockIdx.x;
    float* xr = x + (size_t)r * n;
    const float* yr = y + (size_t)r * n;
    if (n <= JOIN_THREADS * JOIN_KEPT) {
        float vx[JOIN_KEPT], vy[JOIN_KEPT], wj[JOIN_KEPT], wn[JOIN_KEPT];
#pragma unroll
        for (int e = 0; e < JOIN_KEPT; ++e) {
            const int i = threadIdx.x + e * JOIN_THREADS;
            const bool in = i < n;
            vy[e] = in ? yr[i] : 0.0f;
            vx[e] = in ? xr[i] : 0.0f;
            wj[e] = in ? w_join[i] : 0.0f;
            wn[e] = in ? w_next[i] : 0.0f;
        }
        float sq = 0.0f;
#pragma unroll
        for (int e = 0; e < JOIN_KEPT; ++e) sq = fmaf(vy[e], vy[e], sq);
        const float scale_y = 1.0f / sqrtf(block_sum<JOIN_THREADS / 64>(sq, scratch) / (float)n + eps_join);
        sq = 0.0f;
#pragma unroll
        for (int e = 0; e < JOIN_KEPT; ++e) {
            vx[e] = vx[e] + vy[e] * (scale_y * wj[e]);      // an element past the end stays 0
            sq = fmaf(vx[e], vx[e], sq);
        }
        const float scale_x = 1.0f / sqrtf(block_sum<JOIN_THREADS / 64>(sq, scratch) / (float)n + eps_next);
#pragma unroll
        for (int e = 0; e < JOIN_KEPT; ++e) {
            const int i = threadIdx.x + e * JOIN_THREADS;
            if (i < n) {
                xr[i] = vx[e];
                const float h = vx[e] * (scale_x * wn[e]);
                if (out) st(out + (size_t)r * n + i, h);
                if (out32) out32[(size_t)r * n + i] = h;
            }
        }
        return;
    }
    float sq = 0.0f;
    for (int i = threadIdx.x; i < n; i += JOIN_THREADS) sq = fmaf(yr[i], yr[i], sq);
    const float scale_y = 1.0f / sqrtf(block_sum<JOIN_THREADS / 64>(sq, scratch) / (float)n + eps_join);
    sq = 0.0f;
    for (int i = threadIdx.x; i < n; i += JOIN_THREADS) {      // a thread reads back only what it wrote
        const float v = xr[i] + yr[i] * (scale_y * w_join[i]);
        xr[i] = v;
        sq = fmaf(v, v, sq);
    }
    const float scale_x = 1.0f / sqrtf(block_sum<JOIN_THREADS / 64>(sq, scratch) / (float)n + eps_next);
    for (int i = threadIdx.x; i < n; i += JOIN_THREADS) {
        const float h = xr[i] * (scale_x * w_next[i]);
        if (out) st(out + (size_t)r * n + i, h);
        if (out32) out32[(size_t)r * n + i] = h;
    }
}

extern "C" int llmx_rmsnorm_add_norm(float* x, const float* y, const float* w_join, float eps_join, const float* w_next, float eps_next,
                                     void* out, int out_dtype, float* out32, int rows, int n, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (!w_join || !w_next || (!out && !out32)) return -2;
    llmx_note_launch(LK_RMSNORM_ADD_NORM);
    if (out_dtype == LLMX_F32)
        hipLaunchKernelGGL(rmsnorm_add_norm_kernel<float>, dim3(rows), dim3(JOIN_THREADS), 0, stream, x, y, w_join, eps_join, w_next, eps_next,
                           (float*)out, out32, n);
    else
        hipLaunchKernelGGL(rmsnorm_add_norm_kernel<bf16_t>, dim3(rows), dim3(JOIN_THREADS), 0, stream, x, y, w_join, eps_join, w_next, eps_next,
                           (bf16_t*)out, out32, n);
    return LLMX_CHECK_LAUNCH();
}
