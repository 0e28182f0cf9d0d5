// Mixers that carry a matrix state from token to token: for every head a float32 matrix S [D key channels, V value
// channels] in the request's state slot (stored in tiles of 8 value channels, [head][tile][D][8], the last tile padded, so
// that the block that owns a tile reads and writes one run of memory), updated once a token:
//     S <- diag(g_t) S                         (a decay a key channel, acting on S's rows)
//     u  = beta_t (v_t - S^T k_t)              (delta rule; without it u = v_t: gated linear attention)
//     S <- S + k_t u^T,   o_t = S^T q_t        (the read-out sees the token's own write)
// A column of S (one value channel) never meets another, so the scan gives every column to 32 lanes that hold a
// thirty-second of its D values each in registers and walk a request's rows in order: the state after a row is the same bits however
// the rows were cut into steps.  Decays, gates, unit norms and the state are float32 in both number formats.
// Around it: the preparation of a delta-rule row (short causal convolutions with silu, unit-norm q and k, the decay and
// beta), the decay of gated linear attention, and the gated RMS norm of the read-out.
#include "common.h"

__device__ __forceinline__ float sigmoid_ls(float v) { return 1.0f / (1.0f + expf(-v)); }

// ---------------------------------------------------------------------------
// The fused in-projection's row `pre` holds q (G*D) | k (G*D) | v (H*V) at its start and beta's H
// pre-activations at `beta_col`.  Channel c of q | k | v passes a causal convolution over the request's last `taps`
// inputs (weights [C, taps], the last column weighs the row itself): inputs of earlier steps come from the tail the state
// slot keeps ([taps - 1, C] at `tail_off`, oldest first; zero when the request opened), inputs of this step from `pre`.
// Then silu; q and k heads are divided by sqrt(sum of squares + 1e-6); decay = exp(-exp(A_log[h]) softplus(step + dt_bias)).
struct DeltaPrepArgs {
    const float* pre;
    int ld;
    const float* conv_w;
    const float* step_pre;   // [T, H*D] (rows step_ld apart): the decay's projection before its bias
    int step_ld;
    const float* dt_bias;    // [H*D]
    const float* a_log;      // [H]
    const float* state;
    long state_stride;
    int tail_off;
    const int* slot_read;
    const int* row_entry;
    const int* entry_rows;
    float* q;       // [T, G*D]
    float* k;       // [T, G*D]
    float* v;       // [T, H*V]
    float* decay;   // [T, H*D]
    float* beta;    // [T, H]
    int G, H, D, V, taps, beta_col;
};

// One wave a (row, unit): the units of a row are its 2 G heads of q and k (convolution, silu, unit norm), its H heads of
// v (convolution, silu), its H heads of decays, and beta; a unit's values stay in the wave's registers.
#define PREP_MAX 256     // values of a head a wave keeps (4 a lane): the scan's limit on a head's key channels
__device__ __forceinline__ float conv_silu_at(const DeltaPrepArgs& a, const float* __restrict__ tail, int C, int row0, int i, int c) {
    float acc = 0.0f;
    for (int j = 0; j < a.taps; ++j) {
        const int idx = i - (a.taps - 1) + j;
        const float x = idx >= 0 ? a.pre[(size_t)(row0 + idx) * a.ld + c] : tail[(size_t)(a.taps - 1 + idx) * C + c];
        acc = fmaf(a.conv_w[(size_t)c * a.taps + j], x, acc);
    }
    return acc * sigmoid_ls(acc);
}

__global__ void __launch_bounds__(64) delta_prep_kernel(DeltaPrepArgs a) {
    const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int GD = a.G * a.D, HV = a.H * a.V, HD = a.H * a.D;
    const int C = 2 * GD + HV;
    const int e = a.row_entry[t];
    const int row0 = a.entry_rows[2 * e];
    const int i = t - row0;
    const float* tail = a.state + (size_t)a.slot_read[e] * a.state_stride + a.tail_off;
    if (unit < 2 * a.G) {                               // a head of q or k
        const int c0 = unit * a.D;
        float y[PREP_MAX / 64];
        float ss = 0.0f;
#pragma unroll
        for (int u = 0; u < PREP_MAX / 64; ++u) {
            const int d = lane + 64 * u;
            y[u] = d < a.D ? conv_silu_at(a, tail, C, row0, i, c0 + d) : 0.0f;
            ss = fmaf(y[u], y[u], ss);
        }
        const float r = 1.0f / sqrtf(wave_sum(ss) + 1e-6f);
        float* out = unit < a.G ? a.q + (size_t)t * GD + c0 : a.k + (size_t)t * GD + (c0 - GD);
#pragma unroll
        for (int u = 0; u < PREP_MAX / 64; ++u)
            if (lane + 64 * u < a.D) out[lane + 64 * u] = y[u] * r;
    } else if (unit < 2 * a.G + a.H) {                  // a head of v
        const int h = unit - 2 * a.G;
        for (int d = lane; d < a.V; d += 64) a.v[(size_t)t * HV + h * a.V + d] = conv_silu_at(a, tail, C, row0, i, 2 * GD + h * a.V + d);
    } else if (unit < 2 * a.G + 2 * a.H) {              // a head's decays
        const int h = unit - 2 * a.G - a.H;
        const float rate = expf(a.a_log[h]);
        for (int d = lane; d < a.D; d += 64) {
            const int c = h * a.D + d;
            a.decay[(size_t)t * HD + c] = expf(-rate * softplus_f(a.step_pre[(size_t)t * a.step_ld + c] + a.dt_bias[c]));
        }
    } else {
        for (int c = lane; c < a.H; c += 64) a.beta[(size_t)t * a.H + c] = sigmoid_ls(a.pre[(size_t)t * a.ld + a.beta_col + c]);
    }
}

extern "C" int llmx_delta_prep(const float* pre, int ld, const float* conv_w, const float* step_pre, int step_ld, const float* dt_bias,
                               const float* a_log, const float* state, long state_stride, int tail_off, const int* slot_read,
                               const int* row_entry, const int* entry_rows, float* q, float* k, float* v, float* decay, float* beta, int rows, int G,
                               int H, int D, int V, int taps, int beta_col, hipStream_t stream) {
    if (rows <= 0) return 0;
    const long C = 2L * G * D + (long)H * V;
    if (taps < 1 || G < 1 || H % G || D > PREP_MAX || beta_col + H > ld || C > ld || step_ld < H * D) return -2;
    DeltaPrepArgs a{pre, ld, conv_w, step_pre, step_ld, dt_bias, a_log, state, state_stride, tail_off, slot_read, row_entry, entry_rows,
                    q, k, v, decay, beta, G, H, D, V, taps, beta_col};
    llmx_note_launch(LK_DELTA_PREP);
    hipLaunchKernelGGL(delta_prep_kernel, dim3(rows, 2 * G + 2 * H + 1), dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The decay of gated linear attention: out = sigmoid(z + b)^(1 / tau) = exp(-softplus(-(z + b)) / tau), element by element.
__global__ void __launch_bounds__(256) sigmoid_root_kernel(const float* __restrict__ z, const float* __restrict__ bias, float inv_tau,
                                                         float* __restrict__ out, int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    const float x = z[at] + (bias ? bias[(int)(at % (size_t)n)] : 0.0f);
    out[at] = expf(-softplus_f(-x) * inv_tau);
}

extern "C" int llmx_sigmoid_root(const float* z, const float* bias, float inv_tau, float* out, int rows, int n, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    llmx_note_launch(LK_SIGMOID_ROOT);
    const size_t total = (size_t)rows * n;
    hipLaunchKernelGGL(sigmoid_root_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, z, bias, inv_tau, out, n, total);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The scan.  Grid (H * ceil(V / 8), entries), four waves a block: 32 lanes (two rows of 16) own value channel
// 8 * tile + c together, lane s of them the key channels s, 32 + s, ... of its head (R of them).  q and k are read head h / share (several heads may share one), with row
// strides of their own, so they may be columns of a wider projection.  A lane's sums over its R channels run in up to four
// chains (channels i, i + 4, ...: (c0 + c1) + (c2 + c3)); sums over a column's lanes are a butterfly over each row of 16,
// then the two rows' sums added.
// An entry's blocks also hand on the convolution tail, each a share of its channels: the entry's last taps - 1 inputs, from
// this step's rows of `tail_src` and, where the step brought fewer, from the old tail.
struct StateScanArgs {
    const float* q;
    const float* k;
    const float* v;
    const float* decay;
    const float* beta;   // [T, H] or null: no delta correction
    int ldq, ldk, ldv, ldg;
    float* state;
    long state_stride;
    const int* slot_read;
    const int* slot_write;
    const int* entry_rows;
    float* out;          // [T, H*V]
    float out_scale;
    int H, share, D, V;
    const float* tail_src;
    int tail_ld, tail_C, taps, tail_off;
};

// Rows are worked on in chunks of CH: the block brings a chunk's q, k and decay values (its head's D of each, padded to
// 16 R) and its 8 values of v and beta through registers into LDS while the chunk before is worked on, so the chain from
// token to token waits for LDS, not for memory; a token's operands are read from LDS while the token before is worked on.
// Every load is asked for whatever the index (addresses are clamped, the value is chosen afterwards), so none sits behind
// a branch.
__device__ __forceinline__ float column_sum(float v) { return wave_sum(v); }     // over a column's lanes, the same bits in each

#define SCAN_COLS 8     // value channels a block of four waves owns
#define SCAN_LANES 64   // lanes that share a column: a wave
#define SCAN_THREADS (SCAN_COLS * SCAN_LANES)
template <int R, int CH>
__global__ void __launch_bounds__(SCAN_THREADS) state_scan_kernel(StateScanArgs a) {
    constexpr int DP = SCAN_LANES * R;              // a head's key channels, padded
    constexpr int PER_TOKEN = 3 * DP;               // k | q | decay
    constexpr int STAGE = (CH * PER_TOKEN + SCAN_THREADS - 1) / SCAN_THREADS;   // values a thread brings a chunk
    constexpr int NC = R >= 4 ? 4 : R;              // chains a lane's sums run in
    __shared__ __attribute__((aligned(16))) float rows[2][CH][PER_TOKEN];
    __shared__ float vals[2][CH][SCAN_COLS];
    __shared__ float betas[2][CH];
    const int tid = threadIdx.x, s = tid & (SCAN_LANES - 1), c = tid / SCAN_LANES;     // c: 0..7, the block's column; s: the lane's place in it
    const int tiles = (a.V + SCAN_COLS - 1) / SCAN_COLS;
    const int h = blockIdx.x / tiles, tile = blockIdx.x % tiles;
    const int e = blockIdx.y;
    const int row0 = a.entry_rows[2 * e], n = a.entry_rows[2 * e + 1];
    const int j = tile * SCAN_COLS + c;
    const bool col = j < a.V;
    const int d0 = s * R;           // where the lane's operands lie in a staged row; its i-th key channel is 32 i + s
    const size_t slot_r = (size_t)a.slot_read[e] * a.state_stride, slot_w = (size_t)a.slot_write[e] * a.state_stride;

    if (a.taps > 1) {       // the entry's blocks share the tail's channels out among themselves
        const float* old = a.state + slot_r + a.tail_off;
        float* fresh = a.state + slot_w + a.tail_off;
        const int share = (a.tail_C + (int)gridDim.x - 1) / (int)gridDim.x;
        const int ch_end = min(a.tail_C, ((int)blockIdx.x + 1) * share);
        for (int ch = (int)blockIdx.x * share + tid; ch < ch_end; ch += SCAN_THREADS) {
            for (int p = 0; p < a.taps - 1; ++p) {      // ascending: in place, a value is read before its place is written
                const int idx = n - (a.taps - 1) + p;
                fresh[(size_t)p * a.tail_C + ch] = idx >= 0 ? a.tail_src[(size_t)(row0 + idx) * a.tail_ld + ch] : old[(size_t)(n + p) * a.tail_C + ch];
            }
        }
    }

    const int hq = h / a.share;
    const float* kp = a.k + (size_t)hq * a.D;
    const float* qp = a.q + (size_t)hq * a.D;
    const float* gp = a.decay + (size_t)h * a.D;
    const float* vp = a.v + (size_t)h * a.V + tile * SCAN_COLS;
    float stage[STAGE], vstage = 0.0f, bstage = 0.0f;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int idx = min(tid + SCAN_THREADS * u, CH * PER_TOKEN - 1);
            const int tt = idx / PER_TOKEN, rem = idx % PER_TOKEN, which = rem / DP, d = rem % DP;
            const size_t row = (size_t)(row0 + min(t0 + tt, n - 1));
            const int dd = d < a.D ? d : 0;
            const float* src = which == 0 ? kp + row * a.ldk : which == 1 ? qp + row * a.ldq : gp + row * a.ldg;
            const float x = src[dd];
            stage[u] = d < a.D ? x : 0.0f;
        }
        if (tid < CH * SCAN_COLS) {
            const int tt = min(tid / SCAN_COLS, CH - 1), cc = tid % SCAN_COLS;
            vstage = vp[(size_t)(row0 + min(t0 + tt, n - 1)) * a.ldv + min(cc, a.V - 1 - tile * SCAN_COLS)];
        }
        if (a.beta) bstage = a.beta[(size_t)(row0 + min(t0 + min(tid, CH - 1), n - 1)) * a.H + h];
    };
    // a staged row holds channel d at (d % 32) * R + d / 32, so that a lane's R values (channels s, 32 + s, ...) lie together
    auto put = [&](int b) {
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int idx = tid + SCAN_THREADS * u;
            const int tt = idx / PER_TOKEN, rem = idx % PER_TOKEN, which = rem / DP, d = rem % DP;
            if (idx < CH * PER_TOKEN) rows[b][tt][which * DP + (d % SCAN_LANES) * R + d / SCAN_LANES] = stage[u];
        }
        if (tid < CH * SCAN_COLS) (&vals[b][0][0])[tid] = vstage;
        if (tid < CH) betas[b][tid] = bstage;
    };

    fetch(0);
    float S[R];
    const size_t tile_at = ((size_t)h * tiles + tile) * a.D * SCAN_COLS + c;
    {
        const float* src = a.state + slot_r + tile_at;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int d = SCAN_LANES * i + s;
            const float x = src[(size_t)(d < a.D ? d : 0) * SCAN_COLS];
            S[i] = (col && d < a.D) ? x : 0.0f;
        }
    }
    put(0);
    __syncthreads();
    const bool delta = a.beta != nullptr;
    // a token's operands as the lane reads them from the staged chunk; two sets take turns, so that a token's are read while
    // the token before is worked on and nothing is copied from set to set
    struct Operands {
        float k[R], q[R], g[R], v, beta;
    };
    auto read = [&](Operands& x, int b, int tt) {
        const float* kr = &rows[b][tt][d0];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            x.k[i] = kr[i];
            x.q[i] = kr[DP + i];
            x.g[i] = kr[2 * DP + i];
        }
        x.v = vals[b][tt][c];
        x.beta = betas[b][tt];
    };
    const size_t out_ld = (size_t)a.H * a.V;
    // one token: the state's update, and the lane's share of the read-out (summed over the column's lanes later, for a whole
    // chunk at once: only the delta correction's sum lies on the way from a token's state to the next one's)
    auto token = [&](const Operands& x) -> float {
        float u = x.v;
        if (delta) {
            float p[NC];
#pragma unroll
            for (int y = 0; y < NC; ++y) p[y] = 0.0f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                S[i] = S[i] * x.g[i];
                p[i % NC] = fmaf(x.k[i], S[i], p[i % NC]);
            }
            const float dot = NC == 4 ? (p[0] + p[1]) + (p[2] + p[3]) : NC == 2 ? p[0] + p[1] : p[0];
            u = x.beta * (u - column_sum(dot));
        } else {
#pragma unroll
            for (int i = 0; i < R; ++i) S[i] = S[i] * x.g[i];
        }
        float o[NC];
#pragma unroll
        for (int y = 0; y < NC; ++y) o[y] = 0.0f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] = fmaf(x.k[i], u, S[i]);
            o[i % NC] = fmaf(x.q[i], S[i], o[i % NC]);
        }
        return NC == 4 ? (o[0] + o[1]) + (o[2] + o[3]) : NC == 2 ? o[0] + o[1] : o[0];
    };
    Operands first, second;
    float* out_at = a.out + (size_t)row0 * out_ld + (size_t)h * a.V + (col ? j : 0);
    for (int t0 = 0, b = 0; t0 < n; t0 += CH, b ^= 1) {
        // long chunks ask for the next one whatever it is (past the end the last row again, never used): a load behind a
        // branch would be waited for at once; steps of single tokens (CH 2) save the trip
        const bool more = CH > 2 || t0 + CH < n;
        if (more) fetch(t0 + CH);
        const int m = min(CH, n - t0);
        read(first, b, 0);
        float share[CH];
#pragma unroll
        for (int tt = 0; tt < CH; ++tt) {
            if (tt < m) {
                read((tt & 1) ? first : second, b, tt + 1 < CH ? tt + 1 : tt);
                share[tt] = token((tt & 1) ? second : first);
            }
        }
#pragma unroll
        for (int tt = 0; tt < CH; ++tt) {
            if (tt < m) {
                const float sum = column_sum(share[tt]);
                if (s == 0 && col) out_at[(size_t)tt * out_ld] = sum * a.out_scale;
            }
        }
        out_at += (size_t)CH * out_ld;
        if (more) put(b ^ 1);
        __syncthreads();
    }
    {
        float* dst = a.state + slot_w + tile_at;
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (col && SCAN_LANES * i + s < a.D) dst[(size_t)(SCAN_LANES * i + s) * SCAN_COLS] = S[i];
    }
}

extern "C" int llmx_state_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* decay, int ldg,
                               const float* beta, float* state, long state_stride, const int* slot_read, const int* slot_write,
                               const int* entry_rows, float* out, float out_scale, int n_entries, int H, int share, int D, int V,
                               const float* tail_src, int tail_ld, int tail_C, int taps, int tail_off, int max_rows, hipStream_t stream) {
    if (n_entries <= 0) return 0;
    if (H < 1 || share < 1 || H % share || D < 1 || D > 256 || V < 1 || (taps > 1 && !tail_src)) return -2;
    StateScanArgs a{q, k, v, decay, beta, ldq, ldk, ldv, ldg, state, state_stride, slot_read, slot_write, entry_rows, out, out_scale,
                    H, share, D, V, tail_src, tail_ld, tail_C, taps, tail_off};
    const dim3 grid((unsigned)(H * ((V + SCAN_COLS - 1) / SCAN_COLS)), (unsigned)n_entries);
    llmx_note_launch(LK_STATE_SCAN);
    const int per_lane = (D + SCAN_LANES - 1) / SCAN_LANES;
    // steps of single decoded tokens stage chunks of two rows (a quarter of the LDS, so more blocks a compute unit); a
    // row's arithmetic does not depend on the chunk it came in
#define LLMX_SCAN(R_, CH_) \
    do { \
        if (max_rows > 0 && max_rows <= 2) hipLaunchKernelGGL((state_scan_kernel<R_, 2>), grid, dim3(SCAN_THREADS), 0, stream, a); \
        else hipLaunchKernelGGL((state_scan_kernel<R_, CH_>), grid, dim3(SCAN_THREADS), 0, stream, a); \
    } while (0)
    // chunks of 16 rows where LDS holds two of them (heads of at most 128 key channels): a chunk's work then outlasts the
    // next chunk's way from memory
    if (per_lane <= 1) LLMX_SCAN(1, 16);
    else if (per_lane <= 2) LLMX_SCAN(2, 16);
    else LLMX_SCAN(4, 8);
#undef LLMX_SCAN
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// The read-out's gated norm, one wave a (row, head): out = x / sqrt(mean(x^2) + eps) * w * gate(z) * post, gate = sigmoid or
// silu of the gate's pre-activation z (a float32 view with its own row stride; null: no gate); out in the activation type
// for the output projection.  The head's values x come from o, whose heads start `o_head` floats apart:
//   x_j = o_j                                               plainly;
//   x_j = o_j - lambda * o_(sub + j)                        sub > 0: a second map of the head, `sub` floats on, taken off;
//   x_j = o_j / (max(|o_V|, den_floor[t, h]) + 1e-6)        den_floor given: the head's V values are followed by their
//                                                           denominator, which is kept away from zero.
// w: null (no weight), [V] shared by the heads, or (w_wide) [H * V].
enum : int { GATE_SIGMOID = 0, GATE_SILU = 1 };

struct HeadNormArgs {
    const float* o;
    int o_head;
    const float* w;
    int w_wide;
    const float* z;
    int ldz;
    float eps;
    int H, V, gate, sub;
    float lambda, post;
    const float* den_floor;
};

template <typename TO>
__global__ void __launch_bounds__(64) head_norm_gate_kernel(HeadNormArgs a, TO* __restrict__ out) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int H = a.H, V = a.V;
    const float* row = a.o + ((size_t)t * H + h) * a.o_head;
    float den = 1.0f;
    if (a.den_floor) den = fmaxf(fabsf(row[V]), a.den_floor[(size_t)t * H + h]) + 1e-6f;
    auto value = [&](int j) {
        float x = row[j];
        if (a.sub > 0) x = x - a.lambda * row[a.sub + j];
        if (a.den_floor) x = x / den;
        return x;
    };
    float ss = 0.0f;
    for (int j = lane; j < V; j += 64) {
        const float x = value(j);
        ss = fmaf(x, x, ss);
    }
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)V + a.eps);
    const float* zr = a.z ? a.z + (size_t)t * a.ldz + (size_t)h * V : nullptr;
    const float* w = a.w ? (a.w_wide ? a.w + (size_t)h * V : a.w) : nullptr;
    TO* dst = out + ((size_t)t * H + h) * V;
    for (int j = lane; j < V; j += 64) {
        float y = value(j) * r;
        if (w) y = y * w[j];
        if (zr) {
            const float x = zr[j];
            y = y * (a.gate == GATE_SIGMOID ? sigmoid_ls(x) : x * sigmoid_ls(x));
        }
        if (a.post != 1.0f) y = y * a.post;
        st(dst + j, y);
    }
}

extern "C" int llmx_head_norm_gate(const float* o, const float* w, const float* z, int ldz, void* out, int out_dtype, float eps, int rows, int H,
                                   int V, int gate, int o_head, int w_wide, int sub, float lambda, float post, const float* den_floor,
                                   hipStream_t stream) {
    if (rows <= 0) return 0;
    if (H < 1 || V < 1 || (gate != GATE_SIGMOID && gate != GATE_SILU)) return -2;
    if (o_head < V || sub < 0 || (sub > 0 && (den_floor || o_head < sub + V)) || (den_floor && o_head < V + 1)) return -2;
    HeadNormArgs a{o, o_head, w, w_wide, z, ldz, eps, H, V, gate, sub, lambda, post, den_floor};
    llmx_note_launch(LK_HEAD_NORM_GATE);
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(rows, H), dim3(64), 0, stream, a, (float*)out);
    else hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3(rows, H), dim3(64), 0, stream, a, (bf16_t*)out);
    return LLMX_CHECK_LAUNCH();
}

// ---------------------------------------------------------------------------
// A matrix memory with an exponential input gate and a sigmoid forget gate, made ready for the scan above.  Per head and
// token, from the gates' pre-activations zi, zf (with their biases) and a cap c:
//     i_t = c tanh(zi / c),  f_t = log sigmoid(c tanh(zf / c)),  m_t = max(f_t + m_(t-1), i_t)       (m starts at 0)
//     S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t likewise with k_t alone
// which is the scan's recurrence with one decay for all of a head's key channels, keys times exp(i_t - m_t), and one more
// value channel that is always 1 (its column of S is n).  The preparation walks each request's rows in order for m (kept in
// the request's state slot after the matrix, one float a head) and writes the scan's operands: decay [T, H*D], keys
// [T, H*D], values [T, H*(V+1)], and exp(-m_t) [T, H], below which the read-out's denominator |n_t . q_t| is not let.
// Two launches.  The first, one block of 256 threads a (request, head), walks the request's rows in chunks of 256: a chunk's
// gates are formed a thread a row, m by every thread alike in row order, the three exponentials a thread a row; the two
// factors go out as [T, H, 2] (keep, take).  The second, one wave a (row, head), writes the row's operands from them.
struct MemoryPrepArgs {
    const float* pre;        // [T, ld]: the fused projection
    int ld;
    int k_col, v_col, i_col, f_col;
    const float* i_bias;     // [H]
    const float* f_bias;     // [H]
    float cap;
    float* state;
    long state_stride;
    int m_off;
    const int* slot_read;
    const int* slot_write;
    const int* entry_rows;
    float* decay;            // [T, H*D]
    float* keys;             // [T, H*D]
    float* values;           // [T, H*(V+1)]
    float* den_floor;        // [T, H]
    float* factors;          // [T, H, 2]: keep, take
    int H, D, V;
};

#define MEM_CHUNK 256

__global__ void __launch_bounds__(MEM_CHUNK) memory_gates_kernel(MemoryPrepArgs a) {
    __shared__ float gi[MEM_CHUNK], gf[MEM_CHUNK];
    const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int row0 = a.entry_rows[2 * e], n = a.entry_rows[2 * e + 1];
    const int H = a.H;
    float m = a.state[(size_t)a.slot_read[e] * a.state_stride + a.m_off + h];
    const float bi = a.i_bias[h], bf = a.f_bias[h];
    for (int c0 = 0; c0 < n; c0 += MEM_CHUNK) {
        const int rows = min(MEM_CHUNK, n - c0);
        if (tid < rows) {
            const float* r = a.pre + (size_t)(row0 + c0 + tid) * a.ld;
            gi[tid] = a.cap * tanhf((r[a.i_col + h] + bi) / a.cap);
            const float x = a.cap * tanhf((r[a.f_col + h] + bf) / a.cap);
            gf[tid] = -(log1pf(expf(-fabsf(x))) + fmaxf(-x, 0.0f));
        }
        __syncthreads();
        float mine_prev = 0.0f, mine_now = 0.0f;
        for (int t = 0; t < rows; ++t) {        // every thread alike, in row order
            const float now = fmaxf(gf[t] + m, gi[t]);
            if (t == tid) {
                mine_prev = m;
                mine_now = now;
            }
            m = now;
        }
        if (tid < rows) {
            const size_t at = (size_t)(row0 + c0 + tid) * H + h;
            a.factors[2 * at] = expf(gf[tid] + mine_prev - mine_now);
            a.factors[2 * at + 1] = expf(gi[tid] - mine_now);
            a.den_floor[at] = expf(-mine_now);
        }
        __syncthreads();
    }
    if (tid == 0) a.state[(size_t)a.slot_write[e] * a.state_stride + a.m_off + h] = m;
}

__global__ void __launch_bounds__(64) memory_rows_kernel(MemoryPrepArgs a) {
    const size_t row = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const int H = a.H, D = a.D, V = a.V;
    const float* r = a.pre + row * a.ld;
    const float kp = a.factors[2 * (row * H + h)], tk = a.factors[2 * (row * H + h) + 1];
    for (int d = lane; d < D; d += 64) {
        a.decay[(row * H + h) * D + d] = kp;
        a.keys[(row * H + h) * D + d] = tk * r[a.k_col + h * D + d];
    }
    for (int j = lane; j <= V; j += 64) a.values[(row * H + h) * (V + 1) + j] = j < V ? r[a.v_col + h * V + j] : 1.0f;
}

extern "C" int llmx_memory_prep(const float* pre, int ld, int k_col, int v_col, int i_col, int f_col, const float* i_bias, const float* f_bias,
                                float cap, float* state, long state_stride, int m_off, const int* slot_read, const int* slot_write,
                                const int* entry_rows, float* decay, float* keys, float* values, float* den_floor, float* factors, int rows,
                                int n_entries, int H, int D, int V, hipStream_t stream) {
    if (n_entries <= 0 || rows <= 0) return 0;
    if (H < 1 || D < 1 || V < 1 || !(cap > 0.0f) || m_off < 0 || m_off + H > state_stride || !factors) return -2;
    MemoryPrepArgs a{pre, ld, k_col, v_col, i_col, f_col, i_bias, f_bias, cap, state, state_stride, m_off, slot_read, slot_write, entry_rows,
                     decay, keys, values, den_floor, factors, H, D, V};
    llmx_note_launch(LK_MEMORY_PREP);
    hipLaunchKernelGGL(memory_gates_kernel, dim3(n_entries, H), dim3(MEM_CHUNK), 0, stream, a);
    int rc = LLMX_CHECK_LAUNCH();
    if (rc) return rc;
    hipLaunchKernelGGL(memory_rows_kernel, dim3(rows, H), dim3(64), 0, stream, a);
    return LLMX_CHECK_LAUNCH();
}
