// Gated element-wise recurrences over the rows of a step, with a float32 state a request in state slots.
//
// minGRU form: for channel c of a request's rows t = 0 .. n-1 (in position order)
//     z = sigmoid(a[t,c] + bz[c]),  u = b[t,c] + bx[c],  cand = u >= 0 ? u + 1/2 : sigmoid(u),
//     S = (1 - z) * S + z * cand,   out[t,c] = S * silu(g[t,c]),
// where a | b | g are the three thirds of a row of `zxg` (the pre-activations of the gate, the candidate and the output
// gate, float32).  S starts from the request's state slot `slot_read` and ends in `slot_write` (they may be the same):
// a step that computes into a second slot needs no copy of the state first.  One thread owns a channel of a request and
// walks its rows in order, so the state after a row is the same bits however the rows were cut into steps.
#include "common.h"

struct ScanArgs {
    const float* zxg;        // [T, 3W]
    const float* bz;         // [W] or null
    const float* bx;         // [W] or null
    float* state;            // [slots, W]
    const int* slot_read;    // [n_entries]
    const int* slot_write;   // [n_entries]
    const int* entry_rows;   // [n_entries, 2]: first row, rows
    void* out;               // [T, W] in the activation type
    int W;
};


#define SCAN_AHEAD 8
template <typename TO>
__global__ void __launch_bounds__(64) mingru_scan_kernel(ScanArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    const int e = blockIdx.y;
    if (c >= a.W) return;
    const int row0 = a.entry_rows[2 * e], n = a.entry_rows[2 * e + 1];
    const float bz = a.bz ? a.bz[c] : 0.0f, bx = a.bx ? a.bx[c] : 0.0f;
    float S = a.state[(size_t)a.slot_read[e] * a.W + c];
    const size_t ld = 3 * (size_t)a.W;
    TO* out = (TO*)a.out;
    for (int t0 = 0; t0 < n; t0 += SCAN_AHEAD) {
        float za[SCAN_AHEAD], ua[SCAN_AHEAD], ga[SCAN_AHEAD];
        // a round's loads are asked for together; the chain below then runs without waiting for memory
#pragma unroll
        for (int k = 0; k < SCAN_AHEAD; ++k) {
            const int t = t0 + k < n ? t0 + k : n - 1;
            const float* row = a.zxg + (size_t)(row0 + t) * ld;
            za[k] = row[c];
            ua[k] = row[a.W + c];
            ga[k] = row[2 * a.W + c];
        }
#pragma unroll
        for (int k = 0; k < SCAN_AHEAD; ++k) {
            if (t0 + k < n) {
                const float z = sigmoid_f(za[k] + bz);
                const float u = ua[k] + bx;
                const float cand = u >= 0.0f ? u + 0.5f : sigmoid_f(u);
                S = (1.0f - z) * S + z * cand;
                const float g = ga[k];
                st(out + (size_t)(row0 + t0 + k) * a.W + c, S * (g * sigmoid_f(g)));
            }
        }
    }
    a.state[(size_t)a.slot_write[e] * a.W + c] = S;
}

// ---------------------------------------------------------------------------
// The same recurrence for long runs of rows, in three launches over chunks of a request's rows (the host lists them:
// chunks [n, 4] = entry, first row, rows, 1 if it is its entry's last; entry_chunks [n_entries, 2] = first chunk, chunks).
// S_t = a_t S_(t-1) + b_t with a = 1 - z, b = z * cand composes: over a chunk S_end = A S_start + B with A the product of
// its a and B its own recurrence from zero.  (1) every chunk forms (A, B); (2) every request walks its chunks' (A, B)
// from its state and leaves each chunk's S_start; (3) every chunk runs the recurrence from its S_start and stores the
// rows, the last chunk also the state.  A row's value differs from the one-launch form's by rounding only (S_start comes
// through A S + B instead of row by row), which is why short runs keep the one-launch form.
struct ChunkArgs {
    ScanArgs s;
    const int* chunks;
    const int* entry_chunks;
    float* chunk_a;      // [n_chunks, W]
    float* chunk_b;      // [n_chunks, W]; after the second launch: S_start
};

__global__ void __launch_bounds__(64) mingru_chunk_sums_kernel(ChunkArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x, k = blockIdx.y, W = a.s.W;
    if (c >= W) return;
    const int row0 = a.chunks[4 * k + 1], n = a.chunks[4 * k + 2];
    const float bz = a.s.bz ? a.s.bz[c] : 0.0f, bx = a.s.bx ? a.s.bx[c] : 0.0f;
    const size_t ld = 3 * (size_t)W;
    float A = 1.0f, B = 0.0f;
    for (int t0 = 0; t0 < n; t0 += SCAN_AHEAD) {
        float za[SCAN_AHEAD], ua[SCAN_AHEAD];
#pragma unroll
        for (int j = 0; j < SCAN_AHEAD; ++j) {
            const float* row = a.s.zxg + (size_t)(row0 + (t0 + j < n ? t0 + j : n - 1)) * ld;
            za[j] = row[c];
            ua[j] = row[W + c];
        }
#pragma unroll
        for (int j = 0; j < SCAN_AHEAD; ++j)
            if (t0 + j < n) {
                const float z = sigmoid_f(za[j] + bz);
                const float u = ua[j] + bx;
                const float cand = u >= 0.0f ? u + 0.5f : sigmoid_f(u);
                B = (1.0f - z) * B + z * cand;
                A = A * (1.0f - z);
            }
    }
    a.chunk_a[(size_t)k * W + c] = A;
    a.chunk_b[(size_t)k * W + c] = B;
}

__global__ void __launch_bounds__(64) mingru_chunk_starts_kernel(ChunkArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x, e = blockIdx.y, W = a.s.W;
    if (c >= W) return;
    const int k0 = a.entry_chunks[2 * e], nk = a.entry_chunks[2 * e + 1];
    float S = a.s.state[(size_t)a.s.slot_read[e] * W + c];
    for (int k = k0; k < k0 + nk; ++k) {
        const float A = a.chunk_a[(size_t)k * W + c], B = a.chunk_b[(size_t)k * W + c];
        a.chunk_b[(size_t)k * W + c] = S;
        S = A * S + B;
    }
}

template <typename TO>
__global__ void __launch_bounds__(64) mingru_chunk_rows_kernel(ChunkArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x, k = blockIdx.y, W = a.s.W;
    if (c >= W) return;
    const int e = a.chunks[4 * k], row0 = a.chunks[4 * k + 1], n = a.chunks[4 * k + 2], last = a.chunks[4 * k + 3];
    const float bz = a.s.bz ? a.s.bz[c] : 0.0f, bx = a.s.bx ? a.s.bx[c] : 0.0f;
    const size_t ld = 3 * (size_t)W;
    float S = a.chunk_b[(size_t)k * W + c];
    TO* out = (TO*)a.s.out;
    for (int t0 = 0; t0 < n; t0 += SCAN_AHEAD) {
        float za[SCAN_AHEAD], ua[SCAN_AHEAD], ga[SCAN_AHEAD];
#pragma unroll
        for (int j = 0; j < SCAN_AHEAD; ++j) {
            const float* row = a.s.zxg + (size_t)(row0 + (t0 + j < n ? t0 + j : n - 1)) * ld;
            za[j] = row[c];
            ua[j] = row[W + c];
            ga[j] = row[2 * W + c];
        }
#pragma unroll
        for (int j = 0; j < SCAN_AHEAD; ++j)
            if (t0 + j < n) {
                const float z = sigmoid_f(za[j] + bz);
                const float u = ua[j] + bx;
                const float cand = u >= 0.0f ? u + 0.5f : sigmoid_f(u);
                S = (1.0f - z) * S + z * cand;
                const float g = ga[j];
                st(out + (size_t)(row0 + t0 + j) * W + c, S * (g * sigmoid_f(g)));
            }
    }
    if (last) a.s.state[(size_t)a.s.slot_write[e] * W + c] = S;
}

extern "C" int llmx_mingru_scan_chunks(const float* zxg, const float* bz, const float* bx, float* state, const int* slot_read,
                                       const int* slot_write, const int* entry_rows, void* out, int out_dtype, int n_entries, int W,
                                       const int* chunks, int n_chunks, const int* entry_chunks, float* chunk_a, float* chunk_b, hipStream_t stream) {
    if (n_entries <= 0 || W <= 0 || n_chunks <= 0) return 0;
    if (n_chunks > 65535 || n_entries > 65535) return -2;
    llmx_note_launch(LK_GATED_SCAN_CHUNKS);
    ChunkArgs a{ScanArgs{zxg, bz, bx, state, slot_read, slot_write, entry_rows, out, W}, chunks, entry_chunks, chunk_a, chunk_b};
    const unsigned gx = (W + 63) / 64;
    hipLaunchKernelGGL(mingru_chunk_sums_kernel, dim3(gx, n_chunks), dim3(64), 0, stream, a);
    hipLaunchKernelGGL(mingru_chunk_starts_kernel, dim3(gx, n_entries), dim3(64), 0, stream, a);
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(mingru_chunk_rows_kernel<float>, dim3(gx, n_chunks), dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(mingru_chunk_rows_kernel<bf16_t>, dim3(gx, n_chunks), dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}

extern "C" int llmx_mingru_scan(const float* zxg, const float* bz, const float* bx, float* state, const int* slot_read, const int* slot_write,
                                const int* entry_rows, void* out, int out_dtype, int n_entries, int W, hipStream_t stream) {
    if (n_entries <= 0 || W <= 0) return 0;
    if (n_entries > 65535) return -2;
    llmx_note_launch(LK_GATED_SCAN);
    ScanArgs a{zxg, bz, bx, state, slot_read, slot_write, entry_rows, out, W};
    const dim3 grid((W + 63) / 64, n_entries);
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(mingru_scan_kernel<float>, grid, dim3(64), 0, stream, a);
    else hipLaunchKernelGGL(mingru_scan_kernel<bf16_t>, grid, dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}
