// Softmax attention with a sink, a window and a gate for prompts on the matrix cores, bfloat16, compiled for one padded
// key size and one padded value size (PALM_SINK_KK: key size / 32 rounded up; PALM_SINK_VT: value size / 16 rounded up).
//
// A wave owns one or two tiles of 16 consecutive queries of one head; a block is one wave.  For every page of 64 keys that
// some query of the wave sees, the wave computes the transposed scores S^T = K Q^T (keys down, queries across), so that a
// lane's four results of a tile are four keys of ONE query: the softmax statistics of a query then live in the lanes of
// its column, and the weights are already laid out as the B operand of the second product O^T += V^T P^T, whose A operand
// reads runs of keys from the transposed value pages.  Scores leave the matrix cores as 32-bit sums; maximum, exponentials
// (base 2: the scores are scaled by scale * log2 e), sums and the gate are 32-bit; the weights are rounded to bfloat16 for
// the second product, whose sums are 32-bit again.  The sink is a key without a value: a query's running maximum starts at
// the sink's score and its running sum at one.
//
// Layouts as in attention_sink.hip: K [pages, kv_heads, 64, dim], V [pages, kv_heads, vdim, 64].
#include "mfma.h"

#ifndef PALM_SINK_KK
#error "compile with -DPALM_SINK_KK=<ceil(key size / 32)> -DPALM_SINK_VT=<ceil(value size / 16)>"
#endif

PALM_DEFINE_LAST_ERROR()

constexpr int KK = PALM_SINK_KK;
constexpr int VT = PALM_SINK_VT;
// tiles of 16 queries a wave: with two, every key and value fragment that the wave reads feeds twice the products; the
// output tiles of two query tiles fit a lane's registers up to a value size of 256
constexpr int QT = VT <= 16 ? 2 : 1;
constexpr bool V_AHEAD = VT * QT <= 16;                // whether a page's value fragments are all read at its top (registers allowing)
constexpr int SM_QUERIES = 16 * QT;

PALM_API int palm_sink_attention_mfma_sizes(int which) { return which == 0 ? KK * 32 : which == 1 ? VT * 16 : QT; }

__device__ inline bf16x8 load_row8(const bf16_t* row, int col, int dim) {
    // eight values of a row from column `col`; columns beyond `dim` are zero (dim is a multiple of eight).  The read
    // itself is unconditional (of the row's last eight values where the column lies beyond it): no branch around it
    const bf16x8 v = load_bf16x8(row + min(col, dim - 8));
    return col < dim ? v : zero_bf16x8();
}

__global__ __launch_bounds__(WAVE) void sink_attention_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new,
    int heads, int kv_heads, int dim, int vdim, float scale, int window, int has_sink, float sink_score,
    const float* __restrict__ sink_scores, const bf16_t* __restrict__ gate, int gate_stride, int gate_per_head,
    bf16_t* __restrict__ out) {
    const int h = blockIdx.y, b = blockIdx.z;
    if (sink_scores) sink_score = sink_scores[h];                 // a learned score for each head instead of one for all
    const int n_new = seq_new[b];
    const int lane = threadIdx.x;
    // the wave's first query among the sequence's new tokens; the blocks of late queries, which have the most keys before
    // them (without a window), are handed out first, so that the short ones fill in at the end
    const int q0 = (gridDim.x - 1 - blockIdx.x) * SM_QUERIES;
    if (q0 >= n_new) return;
    const int r = lane % 16, g = lane / 16;
    const int start = seq_start[b];
    int qi[QT], qpos[QT], qlow[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        qi[t] = min(q0 + 16 * t + r, n_new - 1);                  // a column beyond the run repeats the last query and stores nothing
        qpos[t] = start + qi[t];
        qlow[t] = window > 0 ? qpos[t] - window + 1 : 0;          // the first key that the query sees (below zero: from the start)
    }
    const int last_pos = start + min(q0 + SM_QUERIES - 1, n_new - 1), first_pos = start + q0;
    const int first_key = window > 0 ? max(0, first_pos - window + 1) : 0;      // the first key that any query of the wave sees
    const int last_low = window > 0 ? last_pos - window + 1 : 0;               // the first key that all of them see
    const float log2e = 1.4426950408889634f;
    const float scale2 = scale * log2e;
    const int kvh = h / (heads / kv_heads);
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    // the queries, as the B operand: column r, eight values of group g for each step of 32 over the key size
    bf16x8 qf[QT][KK];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const bf16_t* qr = q + (((size_t)cu_new[b] + qi[t]) * heads + h) * dim;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[t][kk] = load_row8(qr, kk * 32 + g * 8, dim);
    }
    f32x4 acc[QT][VT];
#pragma unroll
    for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) acc[t][vt] = f32x4{0.f, 0.f, 0.f, 0.f};
    // a query's running sum is kept in parts, one a lane group, added at the end: the sink's one goes to group 0
    float mx[QT], l[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) { mx[t] = has_sink ? sink_score * log2e : -INFINITY; l[t] = has_sink && g == 0 ? 1.f : 0.f; }

    // The key fragments of a page are read one page ahead and the value fragments at the top of their page: both are
    // under way while the matrix cores and the softmax work on what came before.
    bf16x8 kf[4][KK];
    auto read_keys = [&](int pg) {
        const int page = pages[pg];
        const bf16_t* kp = k_cache + ((size_t)page * kv_heads + kvh) * PAGE_TOKENS * dim;
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) kf[n][kk] = load_row8(kp + (size_t)(16 * n + r) * dim, kk * 32 + g * 8, dim);
    };
    const int first_page = first_key / PAGE_TOKENS, last_page = last_pos / PAGE_TOKENS;
    read_keys(first_page);
    for (int pg = first_page; pg <= last_page; ++pg) {
        const int page = pages[pg];
        bf16x8 kc[4][KK];
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) kc[n][kk] = kf[n][kk];
        read_keys(min(pg + 1, last_page));
        const bf16_t* vp = v_cache + ((size_t)page * kv_heads + kvh) * vdim * PAGE_TOKENS;
        auto read_values = [&](int vt, int half) {
            const int vd = 16 * vt + r;
            const bf16_t* vr = vp + (size_t)min(vd, vdim - 1) * PAGE_TOKENS;    // row min(vd, vdim - 1): always there
            const uint2 lo = *reinterpret_cast<const uint2*>(vr + 32 * half + 4 * g);
            const uint2 hi = *reinterpret_cast<const uint2*>(vr + 32 * half + 16 + 4 * g);
            const uint4 both = make_uint4(lo.x, lo.y, hi.x, hi.y);
            return vd < vdim ? __builtin_bit_cast(bf16x8, both) : zero_bf16x8();
        };
        bf16x8 vf[V_AHEAD ? VT : 1][2];
        if constexpr (V_AHEAD) {
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) { vf[vt][0] = read_values(vt, 0); vf[vt][1] = read_values(vt, 1); }
        }
        // the page reaches beyond some query of the wave, or begins before some query's window does
        const bool edge = pg * PAGE_TOKENS + PAGE_TOKENS - 1 > first_pos || pg * PAGE_TOKENS < last_low;
        bf16x8 pf[QT][2];                                          // the weights as B operands: [query tile][32 keys]
        f32x4 s[QT][4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
#pragma unroll
            for (int t = 0; t < QT; ++t) s[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                for (int t = 0; t < QT; ++t) s[t][n] = mfma_16x16x32(kc[n][kk], qf[t][kk], s[t][n]);
        }
        // lane (r, g) holds the keys 16 n + 4 g + i of query r; scores in units of log2: a weight is one exp2 away
#pragma unroll
        for (int t = 0; t < QT; ++t) {
            float top = -INFINITY;
            if (edge) {
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int j = pg * PAGE_TOKENS + 16 * n + 4 * g + i;
                        s[t][n][i] = (j <= qpos[t] && j >= qlow[t]) ? s[t][n][i] * scale2 : -INFINITY;
                        top = fmaxf(top, s[t][n][i]);
                    }
            } else {
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[t][n][i] *= scale2;
                        top = fmaxf(top, s[t][n][i]);
                    }
            }
            top = fmaxf(top, __shfl_xor(top, 16, WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, WAVE));
            const float m_new = fmaxf(mx[t], top);
            // a query that has seen no key yet and sees none in this page (it has no sink, and the page lies before its
            // window): nothing is weighed, and no difference of infinities is made
            const float m_ref = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = exp2f(mx[t] - m_ref);
            mx[t] = m_new;
            float sum = 0.f;
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[t][n][i] = exp2f(s[t][n][i] - m_ref);
                    sum += s[t][n][i];
                }
            l[t] = l[t] * alpha + sum;                             // this lane's part; the groups are added at the end
#pragma unroll
            for (int vt = 0; vt < VT; ++vt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][vt][i] *= alpha;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pf[t][half][i] = (__bf16)s[t][2 * half][i];
                    pf[t][half][4 + i] = (__bf16)s[t][2 * half + 1][i];
                }
        }
        // O^T += V^T P^T: row r of a value tile, the same eight keys of group g as the weights hold
#pragma unroll
        for (int vt = 0; vt < VT; ++vt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const bf16x8 v8 = V_AHEAD ? vf[V_AHEAD ? vt : 0][half] : read_values(vt, half);
#pragma unroll
                for (int t = 0; t < QT; ++t) acc[t][vt] = mfma_16x16x32(v8, pf[t][half], acc[t][vt]);
            }
    }
    // lane (r, g) holds value dimensions 16 vt + 4 g + i of query r
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        l[t] += __shfl_xor(l[t], 16, WAVE);
        l[t] += __shfl_xor(l[t], 32, WAVE);
        const float f = 1.0f / l[t];
        if (q0 + 16 * t + r >= n_new) continue;
        const size_t row = (size_t)cu_new[b] + qi[t];
        bf16_t* op = out + (row * heads + h) * vdim;
        const bf16_t* gp = gate && !gate_per_head ? gate + row * gate_stride + (size_t)h * vdim : nullptr;
        // one gate value for the whole head: its sigmoid goes into the factor that divides by the sum
        const float fh = gate && gate_per_head ? f / (1.0f + __expf(-to_float(gate[row * gate_stride + h]))) : f;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const int vd = 16 * vt + 4 * g;
            if (vd < vdim) {                                        // vdim is a multiple of four
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    o[i] = acc[t][vt][i] * fh;
                    if (gp) o[i] *= 1.0f / (1.0f + __expf(-to_float(gp[vd + i])));
                }
                uint2 w;
                w.x = (uint32_t)f32_to_bf16(o[0]).bits | ((uint32_t)f32_to_bf16(o[1]).bits << 16);
                w.y = (uint32_t)f32_to_bf16(o[2]).bits | ((uint32_t)f32_to_bf16(o[3]).bits << 16);
                *reinterpret_cast<uint2*>(op + vd) = w;
            }
        }
    }
}

PALM_API int palm_sink_attention_mfma(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                      const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                      const int* seq_new, const int* cu_new, int n_seqs, int max_new, int heads, int kv_heads,
                                      int dim, int vdim, float scale, int window, int has_sink, float sink_score,
                                      const float* sink_scores, const void* gate, int gate_stride, int gate_per_head, void* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0,
               "sink_attention_mfma: seqs=%d max_new=%d heads=%d kv=%d dim=%d vdim=%d", n_seqs, max_new, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "sink_attention_mfma: %d heads are not a multiple of %d kv heads", heads, kv_heads);
    PALM_CHECK(dim % 8 == 0 && dim <= KK * 32 && dim > (KK - 1) * 32, "sink_attention_mfma: built for key sizes %d..%d in steps of 8, not %d",
               (KK - 1) * 32 + 8, KK * 32, dim);
    PALM_CHECK(vdim % 4 == 0 && vdim <= VT * 16 && vdim > (VT - 1) * 16, "sink_attention_mfma: built for value sizes %d..%d in steps of 4, not %d",
               (VT - 1) * 16 + 4, VT * 16, vdim);
    PALM_CHECK(max_pages > 0 && window >= 0, "sink_attention_mfma: max_pages %d, window %d", max_pages, window);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(heads <= 65535 && n_seqs <= 65535, "sink_attention_mfma: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    dim3 grid((max_new + SM_QUERIES - 1) / SM_QUERIES, heads, n_seqs);
    sink_attention_mfma_kernel<<<grid, WAVE, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, seq_slot, seq_start, seq_new,
        cu_new, heads, kv_heads, dim, vdim, scale, window, has_sink, sink_score, sink_scores, (const bf16_t*)gate, gate_stride, gate_per_head,
        (bf16_t*)out);
    PALM_LAUNCHED();
    return 0;
}
