// Paged attention with score and visibility rules on the matrix cores (bfloat16 cache, pages of a multiple of 16 tokens,
// head_dim a multiple of 8, value width a multiple of 16).
//
// What the universal kernel of attention.hip computes a (row, head, map) at a time, for rules the plain causal kernels do
// not know: a window that also keeps a request's first keys, chunks of positions, a soft cap on the scores, a distance
// penalty a head, a sink in the softmax's denominator, several score maps a head over one set of values, values of their
// own width, a gate a value.  A column is a (row, head, map); a wave works on a tile of up to 16 columns: consecutive rows
// of one request, one map, and the query heads that read one key/value head (see the kernel).
//
// Keys are grouped in fixed segments of 128 absolute positions, a segment in 4 chunks of 32.  Per column and chunk:
//   scores^T[key][col] = K_tile[16 keys x D] . Q^T[D x 16 cols]    (A = K, B = Q in registers), two tiles of 16 keys
//   the rules; an online softmax over the segment's chunks in key order (float32)
//   o^T[dim][col] += V^T[16 dims x 32 keys] . P^T[32 keys x 16 cols]
// The value pages are stored transposed, and a chunk's keys are dealt to the rows of its two score tiles (key 8a + 4u + b
// in row 4a + b of tile u) so that the 8 weights a lane holds belong to 8 consecutive keys: they are the value product's
// operand as they are.  A chunk or a segment that holds no key a column sees leaves the column's sums as they are, bit
// for bit, so a column does not see which other columns share its tile.  The segments' (m, l, o) are folded in key order
// with one formula; a decoded row's long context is shared out over several items that write their segments' (m, l, o),
// which a second kernel folds in the same order with the same formula: the same bits however the context was shared out.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define AR_SEG 128
#define AR_CHUNKS (AR_SEG / 32)
#define AR_ITEM_INTS 8
#define AR_MERGE_MAX 256    // segments whose maxima and sums the merge holds at a time

struct RulesArgs {
    const bf16_t* q;        // [T, heads * maps, D]
    const bf16_t* k_cache;  // [pages][kv_heads * maps][page_tokens][D]
    const bf16_t* v_cache;  // [pages][kv_heads][VD][page_tokens]
    const int* pos;
    const int* row_entry;
    const int* tables;
    const int* items;       // [n][8]: row0, rows, first head, split, splits, first partial slot (-1: the item stores its result), map, 0
    void* out;              // [T, heads * maps * VD], bfloat16 or float32
    int out_f32;
    float* part_o;          // [slots][VD]
    float* part_ml;         // [slots][2]
    float scale, softcap;
    int n_heads, n_kv_heads, maps, D, VD, page_tokens, max_blocks;
    int window, keep_first, chunk;
    const float* slopes;    // [heads] or null
    const float* sink;      // [heads] or null
    const float* gate;      // null, or logits with row stride gate_ld: one a (row, head) or (gate_wide) one a (row, head, value dim)
    int gate_ld, gate_wide;
    int hpc;                // query heads of a tile's columns: those of one key/value head where their number divides 16, else 1
};

// The lowest position, beyond the kept first ones, that a row at position p sees.
__device__ __forceinline__ int lowest_seen(int p, int window, int chunk) {
    int lo = 0;
    if (window > 0 && p - window + 1 > 0) lo = p - window + 1;
    if (chunk > 0) lo = max(lo, (p / chunk) * chunk);
    return lo;
}

// The segments rows at positions first .. last (of one request) see between them: [0, a_end) and [b_begin, b_end).
struct SegRanges {
    int a_end, b_begin, b_end;
    __device__ __forceinline__ int count() const { return a_end + b_end - b_begin; }
    __device__ __forceinline__ int segment(int ord) const { return ord < a_end ? ord : b_begin + (ord - a_end); }
};
__device__ __forceinline__ SegRanges seg_ranges(int first, int last, int window, int keep_first, int chunk) {
    const int lo = lowest_seen(first, window, chunk);
    const int kept = min(keep_first, lo);
    SegRanges r;
    r.a_end = (kept + AR_SEG - 1) / AR_SEG;
    r.b_begin = max(lo / AR_SEG, r.a_end);
    r.b_end = last / AR_SEG + 1;
    return r;
}

__device__ __forceinline__ float folded_r(float state, float a, float value, float b) { return fmaf(state, a, value * b); }
// state (M, L, O) folded with a segment's (m, l, o): the factors on both.  A segment without a seen key changes nothing.
__device__ __forceinline__ void fold_weights_r(float M, float m, float& a, float& b, float& Mn) {
    Mn = fmaxf(M, m);
    if (Mn == -INFINITY) {
        a = 1.0f;
        b = 0.0f;
    } else {
        a = __expf(M - Mn);
        b = __expf(m - Mn);
    }
}

// tanh as 1 - 2 / (e^2x + 1) with the fast exponential: a few instructions where the library's routine takes tens; its
// absolute error of about 1e-7 (times the cap, on a score) is far below what the bfloat16 operands carry.
__device__ __forceinline__ float tanh_fast(float x) { return 1.0f - __fdividef(2.0f, __expf(2.0f * x) + 1.0f); }

__device__ __forceinline__ int chunk_key_r(int u, int r) { return 8 * (r >> 2) + 4 * u + (r & 3); }

// The last step of a column: the sink joins the denominator, then result = o / l, times the gate.
struct Finish {
    float inv, head_factor;
    __device__ __forceinline__ Finish(const RulesArgs& a, int row, int h, float M, float L) {
        float shrink = 1.0f;
        if (a.sink) {
            const float sk = a.sink[h];
            const float top = fmaxf(M, sk);
            shrink = __expf(M - top);
            L = L * shrink + __expf(sk - top);
        }
        inv = shrink / L;
        head_factor = (a.gate && !a.gate_wide) ? sigmoid_f(a.gate[(size_t)row * a.gate_ld + h]) : 1.0f;
    }
    __device__ __forceinline__ float operator()(const RulesArgs& a, int row, int h, int d, float o) const {
        float y = o * inv;
        if (a.gate) y = y * (a.gate_wide ? sigmoid_f(a.gate[(size_t)row * a.gate_ld + (size_t)h * a.VD + d]) : head_factor);
        return y;
    }
};

// A tile's 16 columns are `hpc` query heads (those that read one key/value head, where their number divides 16; else one
// head) for each of 16 / hpc consecutive rows: column c is row c / hpc of the tile, head h0 + c % hpc.  The keys and values
// a chunk brings are then multiplied for all of a key/value head's query heads at once.
// A segment's page ids are read once (lane i holds the i-th page the segment touches) and handed round by lane index; the
// next chunk's keys and values are asked for before this chunk's are multiplied.
template <int QS, int DT>
__global__ void __launch_bounds__(64) attention_rules_kernel(RulesArgs a) {
    const int* item = a.items + (size_t)blockIdx.x * AR_ITEM_INTS;
    const int row0 = item[0], n_rows = item[1], h0 = item[2], split = item[3], n_splits = item[4], part_base = item[5], map = item[6];
    const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;
    const int M = a.maps, D = a.D, VD = a.VD, PT = a.page_tokens, hpc = a.hpc;
    const int r_c = c / hpc, h = h0 + c % hpc, hm = h * M + map;
    const int kvh = h0 / (a.n_heads / a.n_kv_heads);
    const int key_heads = a.n_kv_heads * M, key_head = kvh * M + map;
    const int qs = (D + 31) / 32, dts = VD / 16;
    const int p0 = a.pos[row0];
    const int p_last = p0 + n_rows - 1;
    const int* table = a.tables + (size_t)a.row_entry[row0] * a.max_blocks;
    const bool col_in = r_c < n_rows;
    const int p_c = p0 + r_c;
    const int lo_c = lowest_seen(p_c, a.window, a.chunk);
    const int lo_min = lowest_seen(p0, a.window, a.chunk);
    const int kept_min = min(a.keep_first, lo_min);
    const float slope = (a.slopes && col_in) ? a.slopes[h] : 0.0f;
    const int hi_c = col_in ? p_c : -1;        // the highest position the column sees
    const float inv_cap = a.softcap > 0.0f ? 1.0f / a.softcap : 0.0f;

    // the columns' queries: lane (c, g) holds dims 32 s + 8 g .. of column c
    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (s < qs && col_in && 32 * s + 8 * g + 8 <= D)
            v = *(const u32x4_t*)(a.q + ((size_t)(row0 + r_c) * a.n_heads * M + hm) * D + 32 * s + 8 * g);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }

    const SegRanges ranges = seg_ranges(p0, p_last, a.window, a.keep_first, a.chunk);
    const int n_ord = ranges.count();
    const int per = (n_ord + n_splits - 1) / n_splits;
    const int ord_begin = split * per, ord_end = min(n_ord, ord_begin + per);

    float Mt = -INFINITY, Lt = 0.0f;
    f32x4_t Ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) Ot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    for (int ord = ord_begin; ord < ord_end; ++ord) {
        const int seg = ranges.segment(ord);
        const int seg0 = seg * AR_SEG;
        // the pages the segment touches (at most 9 for pages of 16 tokens): lane i holds the i-th
        const int first_page = seg0 / PT;
        const int my_page = (lane < 17 && first_page + lane < a.max_blocks) ? table[first_page + lane] : -1;
        auto page_of = [&](int key) { return __shfl(my_page, key / PT - first_page); };
        const int n_ch = min(AR_CHUNKS, (p_last - seg0) / 32 + 1);
        auto next_chunk = [&](int ch) {     // the next chunk from ch on that some column may see keys of
            while (ch < n_ch && seg0 + 32 * ch + 32 <= lo_min && seg0 + 32 * ch >= kept_min) ++ch;
            return ch;
        };
        auto load_chunk = [&](int ch, u32x4_t (&kf)[2][QS], u32x4_t (&vf)[DT]) {
            const int j0 = seg0 + 32 * ch;
            const int key0 = j0 + chunk_key_r(0, c), key1 = j0 + chunk_key_r(1, c), keyv = j0 + 8 * g;
            int page0 = page_of(key0), page1 = page_of(key1), pagev = page_of(keyv);
            if (key0 > p_last) page0 = -1;
            if (key1 > p_last) page1 = -1;
            if (keyv > p_last) pagev = -1;
            const bf16_t* k0 = a.k_cache + (((size_t)max(page0, 0) * key_heads + key_head) * PT + key0 % PT) * D + 8 * g;
            const bf16_t* k1 = a.k_cache + (((size_t)max(page1, 0) * key_heads + key_head) * PT + key1 % PT) * D + 8 * g;
            // values: lane (r = c, g) holds dim 16 dt + r, keys j0 + 8 g .. + 7 (one run of a transposed page)
            const bf16_t* vbase = a.v_cache + (((size_t)max(pagev, 0) * a.n_kv_heads + kvh) * VD + c) * PT + keyv % PT;
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                kf[0][s] = u32x4_t{0u, 0u, 0u, 0u};
                kf[1][s] = u32x4_t{0u, 0u, 0u, 0u};
                if (s < qs && 32 * s + 8 * g + 8 <= D) {
                    if (page0 >= 0) kf[0][s] = *(const u32x4_t*)(k0 + 32 * s);
                    if (page1 >= 0) kf[1][s] = *(const u32x4_t*)(k1 + 32 * s);
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                vf[dt] = u32x4_t{0u, 0u, 0u, 0u};
                if (dt < dts && pagev >= 0) vf[dt] = *(const u32x4_t*)(vbase + (size_t)16 * dt * PT);
            }
        };
        float m = -INFINITY, l = 0.0f;
        f32x4_t o[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // one chunk: its keys and values are in (kf, vf); the following chunk's are asked for into (kf_next, vf_next) first
        auto work = [&](int ch, int following, const u32x4_t (&kf)[2][QS], const u32x4_t (&vf)[DT], u32x4_t (&kf_next)[2][QS], u32x4_t (&vf_next)[DT]) {
            if (following < n_ch) load_chunk(following, kf_next, vf_next);
            const int j0 = seg0 + 32 * ch;
            // scores of the chunk's two tiles
            f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                if (s < qs) {
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kf[0][s]), qf[s], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kf[1][s]), qf[s], s1, 0, 0, 0);
                }
            }
            // the lane's 8 scores: keys j0 + 8 g + 0 .. 7 of column c
            float x[8];
            float cmax = -INFINITY;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int j = j0 + 8 * g + i;
                float v = (i < 4 ? s0[i] : s1[i - 4]) * a.scale;
                if (a.softcap > 0.0f) v = a.softcap * tanh_fast(v * inv_cap);
                if (a.slopes) v = v - slope * (float)(p_c - j);
                const bool seen = j <= hi_c && (j >= lo_c || j < a.keep_first);
                x[i] = seen ? v : -INFINITY;
                cmax = fmaxf(cmax, x[i]);
            }
            cmax = rows_max4(cmax);
            const float m_new = fmaxf(m, cmax);
            float corr = 1.0f, w[8], lsum = 0.0f;
            if (m_new == -INFINITY) {
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = 0.0f;
            } else {
                corr = __expf(m - m_new);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    w[i] = __expf(x[i] - m_new);      // 0 for a key that is not seen
                    lsum += w[i];
                }
            }
            lsum = rows_sum4(lsum);
            l = fmaf(l, corr, lsum);
            m = m_new;
            bf16x8_t pf;
#pragma unroll
            for (int i = 0; i < 8; ++i) pf[i] = (__bf16)w[i];
            const bool rescale = __any(corr != 1.0f);     // o * 1 is o: where no column's maximum moved, the products are left out
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if (dt < dts) {
                    if (rescale) o[dt] = f32x4_t{o[dt][0] * corr, o[dt][1] * corr, o[dt][2] * corr, o[dt][3] * corr};
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vf[dt]), pf, o[dt], 0, 0, 0);
                }
            }
        };
        // two sets of operand registers take turns
        u32x4_t kf_a[2][QS], vf_a[DT], kf_b[2][QS], vf_b[DT];
        int ch = next_chunk(0);
        if (ch < n_ch) load_chunk(ch, kf_a, vf_a);
        while (ch < n_ch) {
            int following = next_chunk(ch + 1);
            work(ch, following, kf_a, vf_a, kf_b, vf_b);
            ch = following;
            if (ch >= n_ch) break;
            following = next_chunk(ch + 1);
            work(ch, following, kf_b, vf_b, kf_a, vf_a);
            ch = following;
        }
        if (part_base >= 0) {       // a decoded row: its columns' sums of the segment go out as they are
            if (c < hpc) {
                const size_t slot = (size_t)part_base + (size_t)ord * hpc + c;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    if (dt < dts) *(f32x4_t*)(a.part_o + slot * VD + 16 * dt + 4 * g) = o[dt];
                if (g == 0) {
                    a.part_ml[2 * slot] = m;
                    a.part_ml[2 * slot + 1] = l;
                }
            }
        } else {
            float fa, fb, Mn;
            fold_weights_r(Mt, m, fa, fb, Mn);
            Lt = folded_r(Lt, fa, l, fb);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                if (dt < dts)
                    Ot[dt] = f32x4_t{folded_r(Ot[dt][0], fa, o[dt][0], fb), folded_r(Ot[dt][1], fa, o[dt][1], fb),
                                     folded_r(Ot[dt][2], fa, o[dt][2], fb), folded_r(Ot[dt][3], fa, o[dt][3], fb)};
            Mt = Mn;
        }
    }
    if (part_base >= 0 || !col_in) return;
    const int row = row0 + r_c;
    const Finish fin(a, row, h, Mt, Lt);
    const size_t at = ((size_t)row * a.n_heads * M + hm) * VD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        if (dt < dts) {
            const int d = 16 * dt + 4 * g;
            const float y0 = fin(a, row, h, d, Ot[dt][0]), y1 = fin(a, row, h, d + 1, Ot[dt][1]), y2 = fin(a, row, h, d + 2, Ot[dt][2]),
                        y3 = fin(a, row, h, d + 3, Ot[dt][3]);
            if (a.out_f32) {
                *(f32x4_t*)((float*)a.out + at + d) = f32x4_t{y0, y1, y2, y3};
            } else {
                bf16_t* dst = (bf16_t*)a.out + at + d;
                st(dst, y0);
                st(dst + 1, y1);
                st(dst + 2, y2);
                st(dst + 3, y3);
            }
        }
    }
}

// The form for prompt portions: a workgroup of four waves takes four tiles of consecutive rows (the same key/value head and
// map), which see nearly the same keys: the workgroup brings each chunk's keys and values from memory once, into LDS (the
// next chunk's travel through registers while this one is multiplied, two LDS buffers take turns, one barrier a chunk), and
// every wave reads its operands from there.  All four waves walk the chunks the workgroup's rows see between them; a chunk
// a wave's columns see nothing of leaves their sums as they are, so a row has the bits the one-wave form gives it.
// Key rows and value rows in LDS are 16 bytes longer than their data, which spreads a read's 16 rows over the banks.
template <int QS, int DT>
__global__ void __launch_bounds__(256) attention_rules_shared_kernel(RulesArgs a, const int* __restrict__ group_items) {
    constexpr int KROW = 64 * QS + 16, VROW = 80;
    constexpr int KBYTES = 32 * KROW, VBYTES = 16 * DT * VROW;
    constexpr int KV = (QS + 1) / 2, VV = (DT + 3) / 4;      // 16-byte pieces of a chunk's keys and values a thread brings
    __shared__ __attribute__((aligned(16))) unsigned char lds[2][KBYTES + VBYTES];
    const int* item = group_items + (size_t)blockIdx.x * AR_ITEM_INTS;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 15, g = lane >> 4;
    const int M = a.maps, D = a.D, VD = a.VD, PT = a.page_tokens, hpc = a.hpc;
    const int tile_rows = 16 / hpc;
    const int group_row0 = item[0], group_rows = item[1], h0 = item[2], map = item[6];
    const int row0 = group_row0 + wave * tile_rows;
    const int n_rows = max(0, min(tile_rows, group_rows - wave * tile_rows));
    const int r_c = c / hpc, h = h0 + c % hpc, hm = h * M + map;
    const int kvh = h0 / (a.n_heads / a.n_kv_heads);
    const int key_heads = a.n_kv_heads * M, key_head = kvh * M + map;
    const int qs = (D + 31) / 32, dts = VD / 16;
    const int gp0 = a.pos[group_row0];
    const int p_last = gp0 + group_rows - 1;               // the workgroup's last row
    const int* table = a.tables + (size_t)a.row_entry[group_row0] * a.max_blocks;
    const bool col_in = r_c < n_rows;
    const int p_c = gp0 + wave * tile_rows + r_c;
    const int lo_c = lowest_seen(p_c, a.window, a.chunk);
    const int lo_min = lowest_seen(gp0, a.window, a.chunk);
    const int kept_min = min(a.keep_first, lo_min);
    const float slope = (a.slopes && col_in) ? a.slopes[h] : 0.0f;
    const int hi_c = col_in ? p_c : -1;
    const float inv_cap = a.softcap > 0.0f ? 1.0f / a.softcap : 0.0f;

    bf16x8_t qf[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (s < qs && col_in && 32 * s + 8 * g + 8 <= D)
            v = *(const u32x4_t*)(a.q + ((size_t)(row0 + r_c) * a.n_heads * M + hm) * D + 32 * s + 8 * g);
        qf[s] = __builtin_bit_cast(bf16x8_t, v);
    }
    const SegRanges ranges = seg_ranges(gp0, p_last, a.window, a.keep_first, a.chunk);
    const int n_ord = ranges.count();
    const int kparts = D / 8;      // 16-byte pieces of a key row

    float Mt = -INFINITY, Lt = 0.0f;
    f32x4_t Ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) Ot[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // The chunks some row of the workgroup may see keys of, in key order over all segments: (segment's place, chunk in it).
    auto settle = [&](int& ord, int& ch) {      // the first such chunk at or after (ord, ch); ord = n_ord when none is left
        while (ord < n_ord) {
            const int seg0 = ranges.segment(ord) * AR_SEG;
            const int n_ch = min(AR_CHUNKS, (p_last - seg0) / 32 + 1);
            while (ch < n_ch && seg0 + 32 * ch + 32 <= lo_min && seg0 + 32 * ch >= kept_min) ++ch;
            if (ch < n_ch) return;
            ++ord;
            ch = 0;
        }
    };
    // the thread's pieces of a chunk, from memory into registers ...
    auto fetch = [&](int ord, int ch, u32x4_t (&kr)[KV], u32x4_t (&vr)[VV]) {
        const int j0 = ranges.segment(ord) * AR_SEG + 32 * ch;
#pragma unroll
        for (int u = 0; u < KV; ++u) {
            const int i = tid + 256 * u;
            const int key = j0 + i / kparts, part = i % kparts;
            const int page = (key <= p_last && i < 32 * kparts) ? table[key / PT] : -1;
            kr[u] = u32x4_t{0u, 0u, 0u, 0u};
            if (page >= 0) kr[u] = *(const u32x4_t*)(a.k_cache + (((size_t)page * key_heads + key_head) * PT + key % PT) * D + 8 * part);
        }
#pragma unroll
        for (int u = 0; u < VV; ++u) {
            const int i = tid + 256 * u;
            const int dim = i >> 2, keyv = j0 + 8 * (i & 3);
            const int page = (keyv <= p_last && dim < VD) ? table[keyv / PT] : -1;
            vr[u] = u32x4_t{0u, 0u, 0u, 0u};
            if (page >= 0) vr[u] = *(const u32x4_t*)(a.v_cache + (((size_t)page * a.n_kv_heads + kvh) * VD + dim) * PT + keyv % PT);
        }
    };
    // ... and from there into an LDS buffer
    auto put = [&](int buf, const u32x4_t (&kr)[KV], const u32x4_t (&vr)[VV]) {
#pragma unroll
        for (int u = 0; u < KV; ++u) {
            const int i = tid + 256 * u;
            if (i < 32 * kparts) *(u32x4_t*)(lds[buf] + (i / kparts) * KROW + 16 * (i % kparts)) = kr[u];
        }
#pragma unroll
        for (int u = 0; u < VV; ++u) {
            const int i = tid + 256 * u;
            if ((i >> 2) < VD) *(u32x4_t*)(lds[buf] + KBYTES + (i >> 2) * VROW + 16 * (i & 3)) = vr[u];
        }
    };
    float m = -INFINITY, l = 0.0f;
    f32x4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    int buf = 0;
    // one chunk from the LDS buffer `buf`
    auto work = [&](int ord, int ch) {
        if (n_rows <= 0) return;
        const int j0 = ranges.segment(ord) * AR_SEG + 32 * ch;
        const unsigned char* kb = lds[buf];
        const unsigned char* vb = lds[buf] + KBYTES;
        f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            if (s < qs) {
                u32x4_t x0 = {0u, 0u, 0u, 0u}, x1 = {0u, 0u, 0u, 0u};
                if (32 * s + 8 * g + 8 <= D) {
                    x0 = *(const u32x4_t*)(kb + chunk_key_r(0, c) * KROW + 64 * s + 16 * g);
                    x1 = *(const u32x4_t*)(kb + chunk_key_r(1, c) * KROW + 64 * s + 16 * g);
                }
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x0), qf[s], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x1), qf[s], s1, 0, 0, 0);
            }
        }
        float x[8];
        float cmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int j = j0 + 8 * g + i;
            float v = (i < 4 ? s0[i] : s1[i - 4]) * a.scale;
            if (a.softcap > 0.0f) v = a.softcap * tanh_fast(v * inv_cap);
            if (a.slopes) v = v - slope * (float)(p_c - j);
            const bool seen = j <= hi_c && (j >= lo_c || j < a.keep_first);
            x[i] = seen ? v : -INFINITY;
            cmax = fmaxf(cmax, x[i]);
        }
        cmax = rows_max4(cmax);
        const float m_new = fmaxf(m, cmax);
        float corr = 1.0f, w[8], lsum = 0.0f;
        if (m_new == -INFINITY) {
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = 0.0f;
        } else {
            corr = __expf(m - m_new);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                w[i] = __expf(x[i] - m_new);
                lsum += w[i];
            }
        }
        lsum = rows_sum4(lsum);
        l = fmaf(l, corr, lsum);
        m = m_new;
        bf16x8_t pf;
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[i] = (__bf16)w[i];
        const bool rescale = __any(corr != 1.0f);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (dt < dts) {
                const u32x4_t vv = *(const u32x4_t*)(vb + (16 * dt + c) * VROW + 16 * g);
                if (rescale) o[dt] = f32x4_t{o[dt][0] * corr, o[dt][1] * corr, o[dt][2] * corr, o[dt][3] * corr};
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vv), pf, o[dt], 0, 0, 0);
            }
        }
    };
    // a segment's sums join the tile's, and the segment's start over
    auto fold = [&]() {
        float fa, fb, Mn;
        fold_weights_r(Mt, m, fa, fb, Mn);
        Lt = folded_r(Lt, fa, l, fb);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (dt < dts)
                Ot[dt] = f32x4_t{folded_r(Ot[dt][0], fa, o[dt][0], fb), folded_r(Ot[dt][1], fa, o[dt][1], fb),
                                 folded_r(Ot[dt][2], fa, o[dt][2], fb), folded_r(Ot[dt][3], fa, o[dt][3], fb)};
            o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
        Mt = Mn;
        m = -INFINITY;
        l = 0.0f;
    };
    // this chunk (o0, c0) is in LDS, the next (o1, c1) is on its way in one set of registers, the one after (o2, c2) is asked
    // for into the other set before this chunk is multiplied; the two sets take turns
    int o0 = 0, c0 = 0;
    settle(o0, c0);
    int o1 = o0, c1 = c0 + 1;
    settle(o1, c1);
    int o2 = o1, c2 = c1 + 1;
    settle(o2, c2);
    u32x4_t kr_a[KV], vr_a[VV], kr_b[KV], vr_b[VV];
    if (o0 < n_ord) {
        fetch(o0, c0, kr_a, vr_a);
        put(0, kr_a, vr_a);
    }
    if (o1 < n_ord) fetch(o1, c1, kr_a, vr_a);
    __syncthreads();
    auto turn = [&](const u32x4_t (&kr_next)[KV], const u32x4_t (&vr_next)[VV], u32x4_t (&kr_after)[KV], u32x4_t (&vr_after)[VV]) {
        if (o2 < n_ord) fetch(o2, c2, kr_after, vr_after);
        work(o0, c0);
        if (o1 != o0) fold();                     // the segment's last chunk (also the last chunk of all: o1 = n_ord)
        if (o1 < n_ord) put(buf ^ 1, kr_next, vr_next);
        __syncthreads();
        buf ^= 1;
        o0 = o1;
        c0 = c1;
        o1 = o2;
        c1 = c2;
        if (o2 < n_ord) {
            ++c2;
            settle(o2, c2);
        }
    };
    while (o0 < n_ord) {
        turn(kr_a, vr_a, kr_b, vr_b);
        if (o0 >= n_ord) break;
        turn(kr_b, vr_b, kr_a, vr_a);
    }
    if (!col_in) return;
    const int row = row0 + r_c;
    const Finish fin(a, row, h, Mt, Lt);
    const size_t at = ((size_t)row * a.n_heads * M + hm) * VD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        if (dt < dts) {
            const int d = 16 * dt + 4 * g;
            const float y0 = fin(a, row, h, d, Ot[dt][0]), y1 = fin(a, row, h, d + 1, Ot[dt][1]), y2 = fin(a, row, h, d + 2, Ot[dt][2]),
                        y3 = fin(a, row, h, d + 3, Ot[dt][3]);
            if (a.out_f32) {
                *(f32x4_t*)((float*)a.out + at + d) = f32x4_t{y0, y1, y2, y3};
            } else {
                bf16_t* dst = (bf16_t*)a.out + at + d;
                st(dst, y0);
                st(dst + 1, y1);
                st(dst + 2, y2);
                st(dst + 3, y3);
            }
        }
    }
}

// Folds the segments' sums of a decoded row's column in key order and stores its result: one wave a (row, head, map),
// lane d owning value dims d, d + 64, ...  merges [n][4]: row, head * maps + map, the column's first partial slot, slots from one
// segment's to the next's.
__global__ void __launch_bounds__(64) attention_rules_merge_kernel(RulesArgs a, const int* __restrict__ merges) {
    const int* mg = merges + (size_t)blockIdx.x * 4;
    const int row = mg[0], hm = mg[1], base = mg[2], stride = mg[3];
    const int lane = threadIdx.x, VD = a.VD, M = a.maps;
    const int h = hm / M;
    const int p = a.pos[row];
    const int n_ord = seg_ranges(p, p, a.window, a.keep_first, a.chunk).count();
    // the segments' maxima and sums first (lane i asks for those of segments i, i + 64, ...), then the value sums with four
    // segments' loads in flight; the fold itself is the tiles' chain, a segment at a time
    __shared__ float ms[AR_MERGE_MAX], ls[AR_MERGE_MAX];
    float Mt = -INFINITY, Lt = 0.0f;
    float O[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int ord0 = 0; ord0 < n_ord; ord0 += AR_MERGE_MAX) {
        const int n = min(AR_MERGE_MAX, n_ord - ord0);
        __syncthreads();
        for (int i = lane; i < n; i += 64) {
            const size_t slot = (size_t)base + (size_t)(ord0 + i) * stride;
            ms[i] = a.part_ml[2 * slot];
            ls[i] = a.part_ml[2 * slot + 1];
        }
        __syncthreads();
        for (int i0 = 0; i0 < n; i0 += 4) {
            float v[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const size_t slot = (size_t)base + (size_t)(ord0 + min(i0 + u, n - 1)) * stride;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = lane + 64 * i;
                    v[u][i] = d < VD ? a.part_o[slot * VD + d] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (i0 + u < n) {
                    float fa, fb, Mn;
                    fold_weights_r(Mt, ms[i0 + u], fa, fb, Mn);
                    Lt = folded_r(Lt, fa, ls[i0 + u], fb);
#pragma unroll
                    for (int i = 0; i < 4; ++i) O[i] = folded_r(O[i], fa, v[u][i], fb);
                    Mt = Mn;
                }
            }
        }
    }
    const Finish fin(a, row, h, Mt, Lt);
    const size_t at = ((size_t)row * a.n_heads * M + hm) * VD;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        if (d < VD) {
            const float y = fin(a, row, h, d, O[i]);
            if (a.out_f32) ((float*)a.out)[at + d] = y;
            else st((bf16_t*)a.out + at + d, y);
        }
    }
}

extern "C" int llmx_attention_rules_ok(int dtype, int head_dim, int v_dim, int page_tokens) {
    return dtype == LLMX_BF16 && head_dim >= 8 && head_dim <= 256 && head_dim % 8 == 0 && v_dim >= 16 && v_dim <= 256 && v_dim % 16 == 0 &&
           page_tokens % 16 == 0;
}

extern "C" int llmx_attention_rules_segment(void) { return AR_SEG; }

// Whether the four-wave form for prompt portions is built for these widths (its LDS buffers fit for heads up to 128 wide).
extern "C" int llmx_attention_rules_shared_ok(int head_dim, int v_dim) { return head_dim <= 128 && v_dim <= 128; }

extern "C" int llmx_attention_rules(const void* q, const void* k_cache, const void* v_cache, const int* pos, const int* row_entry, const int* tables,
                                    const int* items, int n_items, const int* group_items, int n_group_items, const int* merges, int n_merges, void* out, int out_f32, float* part_o,
                                    float* part_ml, float scale, float softcap, int n_heads, int n_kv_heads, int maps, int head_dim, int v_dim,
                                    int page_tokens, int max_blocks, int window, int keep_first, int chunk, const float* slopes, const float* sink,
                                    const float* gate, int gate_ld, int gate_wide, int hpc, hipStream_t stream) {
    if (n_items <= 0 && n_group_items <= 0) return 0;
    if (n_group_items > 0 && (!group_items || !llmx_attention_rules_shared_ok(head_dim, v_dim))) return -2;
    if (!llmx_attention_rules_ok(LLMX_BF16, head_dim, v_dim, page_tokens) || maps < 1 || n_heads % n_kv_heads || window < 0 || keep_first < 0 ||
        chunk < 0 || hpc < 1 || hpc > 16 || 16 % hpc || (hpc > 1 && hpc != n_heads / n_kv_heads) || (n_merges > 0 && (!part_o || !part_ml || !merges)) || (gate && gate_ld < (gate_wide ? n_heads * v_dim : n_heads)))
        return -2;
    RulesArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, pos, row_entry, tables, items, out, out_f32, part_o, part_ml,
                scale, softcap, n_heads, n_kv_heads, maps, head_dim, v_dim, page_tokens, max_blocks, window, keep_first, chunk, slopes, sink,
                gate, gate_ld, gate_wide, hpc};
    const int qs = (head_dim + 31) / 32, dts = v_dim / 16;
    if (n_group_items > 0) {
        llmx_note_launch(LK_ATTENTION_RULES_SHARED);
#define LLMX_SHARED(QS_, DT_) hipLaunchKernelGGL((attention_rules_shared_kernel<QS_, DT_>), dim3(n_group_items), dim3(256), 0, stream, a, group_items)
        if (qs <= 2) {
            if (dts <= 4) LLMX_SHARED(2, 4);
            else LLMX_SHARED(2, 8);
        } else {
            if (dts <= 4) LLMX_SHARED(4, 4);
            else LLMX_SHARED(4, 8);
        }
#undef LLMX_SHARED
        const int rc = LLMX_CHECK_LAUNCH();
        if (rc) return rc;
    }
    if (n_items <= 0) return 0;
    llmx_note_launch(LK_ATTENTION_RULES);
#define LLMX_RULES(QS_, DT_) hipLaunchKernelGGL((attention_rules_kernel<QS_, DT_>), dim3(n_items), dim3(64), 0, stream, a)
    if (qs <= 2) {
        if (dts <= 4) LLMX_RULES(2, 4);
        else if (dts <= 8) LLMX_RULES(2, 8);
        else LLMX_RULES(2, 16);
    } else if (qs <= 4) {
        if (dts <= 4) LLMX_RULES(4, 4);
        else if (dts <= 8) LLMX_RULES(4, 8);
        else LLMX_RULES(4, 16);
    } else {
        if (dts <= 4) LLMX_RULES(8, 4);
        else if (dts <= 8) LLMX_RULES(8, 8);
        else LLMX_RULES(8, 16);
    }
#undef LLMX_RULES
    int rc = LLMX_CHECK_LAUNCH();
    if (rc) return rc;
    if (n_merges > 0) {
        llmx_note_launch(LK_ATTENTION_RULES_MERGE);
        hipLaunchKernelGGL(attention_rules_merge_kernel, dim3(n_merges), dim3(64), 0, stream, a, merges);
        rc = LLMX_CHECK_LAUNCH();
    }
    return rc;
}
