// A matrix memory with an input gate and a forget gate per head and token (the mLSTM of xLSTM), kept relative to a running
// maximum so that its exponentials never overflow.
//
//   i_t = cap tanh(a_t / cap)                      log input gate   (a_t, b_t: the gate rows plus their biases)
//   f_t = logsigmoid(cap tanh(b_t / cap))          log forget gate
//   m_t = max(f_t + m_(t-1), i_t)                  m before the first token is 0
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T         S: [dim, vdim] per sequence and head
//   n_t = the same with k_t alone                                               n: [dim]
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * w * sigmoid(gate_t)              (the unit norm is per head, w over all heads)
//
// S, n and m are 32-bit and kept per sequence; gates, their logarithms, exponentials, the sums over the state and the norm
// are 32-bit whatever the rows' type.  n is stored as one more column of S, so S and n are one tensor [dim, vdim + 1].
//
// Three passes.  `gates`: a wave per (sequence, head) walks over the new tokens 64 at a time; each lane makes its token's
// i and f, the wave composes the maps m -> max(m + f, i) with a scan (they are closed under composition), and every token
// gets its three factors: what S keeps, what it takes, and exp(-m).  `qk`: q (times its scale) and k as 32-bit rows padded
// to the key size the main kernel is compiled for.  The main kernel: one block per (head, sequence), one thread per column
// of S, the thread keeps its column in registers and walks over the tokens; q and k of a token are the same for all
// threads: a wave reads them one value a lane and hands them to its lanes as scalars.  n lies across the lanes of every
// wave the same way (the lane that holds k[d] holds n[d]), so n . q is one multiply-add a lane and a sum over the wave, and
// no thread is spent on it; outputs are finished a tile of tokens at a time.  A prompt and a single token run the
// same code, so a prompt leaves the state that its tokens one by one leave.
//
// Given the factors the recurrence is linear in S, so a long run of new tokens is cut into chunks that run side by side:
//   1. every chunk alone from a zero state: its own sum L_c, and the product of what its tokens keep
//   2. the chunks' starting states, one after the other: S_(c+1) = keep_c S_c + L_c, S_0 the kept state
//   3. every chunk from its starting state, now with outputs
#include "common.h"

constexpr int ML_TILE = 8;

enum MlstmMode : int { ML_WHOLE = 0, ML_LOCAL = 1, ML_FROM_STARTS = 2 };

__device__ inline float ml_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// coef[row][head] = (keep, take, exp(-m), unused).  gates float32 [n, 2 heads]: the input gates' rows, then the forget gates'.
__global__ __launch_bounds__(WAVE) void mlstm_gates_kernel(const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                                                           float* __restrict__ m_state, const int* __restrict__ seq_slot,
                                                           const int* __restrict__ seq_new, const int* __restrict__ cu_new, int heads,
                                                           float4* __restrict__ coef) {
    const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const size_t row0 = (size_t)cu_new[b];
    float* mp = m_state + (size_t)seq_slot[b] * heads + h;
    float m_in = *mp;
    const float bi = gate_bias ? gate_bias[h] : 0.f, bf = gate_bias ? gate_bias[heads + h] : 0.f;
    for (int t0 = 0; t0 < n_new; t0 += WAVE) {
        const int t = t0 + lane;
        const bool live = t < n_new;
        const size_t row = row0 + min(t, n_new - 1);
        const float zi = gates[row * 2 * heads + h] + bi, zf = gates[row * 2 * heads + heads + h] + bf;
        const float gi = cap * tanhf(zi / cap);
        const float gf = ml_logsigmoid(cap * tanhf(zf / cap));
        // the token's map m -> max(m + a, c); a token beyond the run is the identity
        float a = live ? gf : 0.f, c = live ? gi : -INFINITY;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float a_o = __shfl_up(a, off, WAVE), c_o = __shfl_up(c, off, WAVE);
            if (lane >= off) { c = fmaxf(c_o + a, c); a = a_o + a; }          // the earlier tokens' map first, then this one's
        }
        const float m_t = fmaxf(m_in + a, c);
        float m_prev = __shfl_up(m_t, 1, WAVE);
        if (lane == 0) m_prev = m_in;
        if (live) coef[row * heads + h] = make_float4(expf(gf + m_prev - m_t), expf(gi - m_t), expf(-m_t), 0.f);
        m_in = __shfl(m_t, WAVE - 1, WAVE);
    }
    if (lane == 0) *mp = m_in;
}

// qk[row][head][0 = q, 1 = k][pad]: q times q_scale and k, 32-bit, zero beyond dim.
template <typename T>
__global__ void mlstm_qk_kernel(const T* __restrict__ rows, int row_stride, int q_off, int k_off, float q_scale, int n_tokens, int heads,
                                int dim, int pad, float* __restrict__ qk) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)n_tokens * heads * pad) return;
    const int d = (int)(idx % pad), h = (int)((idx / pad) % heads);
    const size_t row = (size_t)(idx / ((long long)pad * heads));
    float* o = qk + ((row * heads + h) * 2) * pad + d;
    if (d >= dim) { o[0] = 0.f; o[pad] = 0.f; return; }
    o[0] = to_float(rows[row * row_stride + q_off + h * dim + d]) * q_scale;
    o[pad] = to_float(rows[row * row_stride + k_off + h * dim + d]);
}

// Thread v owns column v of S.  DMAX: the padded key size; MAXT: the most threads of a block.
template <typename T, int DMAX, int MAXT>
__global__ __launch_bounds__(MAXT) void mlstm_kernel(int mode, int chunk, int max_chunks, float* __restrict__ starts, float* __restrict__ chunk_keep,
                                                     const T* __restrict__ rows, int row_stride, int v_off, int g_off, const float* __restrict__ qk,
                                                     const float4* __restrict__ coef, const float* __restrict__ norm_w, float eps,
                                                     float* __restrict__ state, const int* __restrict__ seq_slot, const int* __restrict__ seq_new,
                                                     const int* __restrict__ cu_new, int heads, int dim, int vdim, T* __restrict__ out) {
    __shared__ float red[ML_TILE][16];
    __shared__ float o_s[ML_TILE][MAXT];
    __shared__ float floor_s[ML_TILE], nq_s[ML_TILE];
    constexpr int QREGS = (DMAX + WAVE - 1) / WAVE;
    const int h = blockIdx.x, b = blockIdx.y / max_chunks, c = blockIdx.y % max_chunks;
    const int v = threadIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const int seq_tokens = seq_new[b];
    if (c * chunk >= seq_tokens) return;
    const int n_new = mode == ML_WHOLE ? seq_tokens : min(chunk, seq_tokens - c * chunk);
    const int row0 = cu_new[b] + (mode == ML_WHOLE ? 0 : c * chunk);
    const int cols = vdim + 1;
    const bool mine = v < vdim;
    float* sp = mode == ML_WHOLE ? state + (((size_t)seq_slot[b] * heads + h) * dim) * cols + v
                                 : starts + ((((size_t)b * max_chunks + c) * heads + h) * dim) * cols + v;

    // the reads are unconditional (of a row and a column that exist) and what does not belong is set to zero after
    float S[DMAX];
    {
        const float* at = sp - v + min(v, vdim - 1);
        const bool zero = mode == ML_LOCAL || !mine;
        if (dim == DMAX) {
            const size_t stride = (size_t)cols;
#pragma unroll
            for (int d = 0; d < DMAX; ++d) S[d] = at[d * stride];
            if (zero) {
#pragma unroll
                for (int d = 0; d < DMAX; ++d) S[d] = 0.f;
            }
        } else {
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float s0 = at[(size_t)min(d, dim - 1) * cols];
                S[d] = (zero || d >= dim) ? 0.f : s0;
            }
        }
    }

    // n: the lane that holds k[d] of a token holds n[d]; every wave keeps a copy
    float nreg[QREGS];
#pragma unroll
    for (int i = 0; i < QREGS; ++i) {
        const int d = i * WAVE + lane;
        const float n0 = (sp - v)[(size_t)min(d, dim - 1) * cols + vdim];
        nreg[i] = (mode == ML_LOCAL || d >= dim) ? 0.f : n0;
    }

    // A token's inputs: the thread's value, its three factors, and of its q and k rows one value a lane, which the wave
    // hands to all its lanes as scalars.  The next token's are read while this one's are used.
    const int vc = min(v, vdim - 1);
    auto read_token = [&](int t, float& vv, float4& f, float (&qv)[QREGS], float (&kv)[QREGS]) {
        const size_t row = (size_t)(row0 + t);
        vv = to_float(rows[row * row_stride + v_off + h * vdim + vc]);
        f = coef[row * heads + h];
        const float* __restrict__ qr = qk + ((row * heads + h) * 2) * DMAX;
#pragma unroll
        for (int i = 0; i < QREGS; ++i) {
            const int at = min(i * WAVE + lane, DMAX - 1);
            qv[i] = qr[at];
            kv[i] = qr[DMAX + at];
        }
    };
    float vv, qv[QREGS], kv[QREGS], kept = 1.f;
    float4 f;
    if (n_new > 0) read_token(0, vv, f, qv, kv);
    for (int t0 = 0; t0 < n_new; t0 += ML_TILE) {
        const int tt = min(ML_TILE, n_new - t0);
        for (int ti = 0; ti < tt; ++ti) {
            float vn, qn[QREGS], kn[QREGS];
            float4 fn;
            read_token(min(t0 + ti + 1, n_new - 1), vn, fn, qn, kn);
            if (!mine) vv = 0.f;
            const float keep = f.x, in = f.y * vv;
            kept *= keep;
            float nq = 0.f;
#pragma unroll
            for (int i = 0; i < QREGS; ++i) {
                nreg[i] = fmaf(keep, nreg[i], f.y * kv[i]);
                if (i * WAVE + lane < DMAX) nq = fmaf(nreg[i], qv[i], nq);        // (a key size below a wave: the upper lanes repeat)
            }
            float acc = 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float qd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, qv[d / WAVE]), d % WAVE));
                const float kd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kv[d / WAVE]), d % WAVE));
                S[d] = fmaf(keep, S[d], kd * in);
                acc = fmaf(S[d], qd, acc);
            }
            if (mode != ML_LOCAL) {
                nq = wave_sum(nq);
                o_s[ti][v] = acc;
                const float ss = wave_sum(acc * acc);
                if (lane == 0) red[ti][wave] = ss;
                if (v == 0) { floor_s[ti] = f.z; nq_s[ti] = nq; }
            }
            vv = vn;
            f = fn;
#pragma unroll
            for (int i = 0; i < QREGS; ++i) { qv[i] = qn[i]; kv[i] = kn[i]; }
        }
        if (mode == ML_LOCAL) continue;
        __syncthreads();
        for (int ti = 0; ti < tt; ++ti) {
            float total = 0.f;
            for (int w = 0; w < n_waves; ++w) total += red[ti][w];
            // o = acc / denom for every column of the head, so the head's sum of squares is the raw one over denom^2
            const float denom = fmaxf(fabsf(nq_s[ti]), floor_s[ti]) + 1e-6f;
            const float inv = 1.0f / sqrtf(total / (denom * denom) / (float)vdim + eps);
            const size_t row = (size_t)(row0 + t0 + ti);
            const float gate = to_float(rows[row * row_stride + g_off + h * vdim + vc]);
            if (mine)
                out[row * ((size_t)heads * vdim) + h * vdim + v] =
                    from_float<T>(o_s[ti][v] / denom * inv * norm_w[h * vdim + v] * (1.0f / (1.0f + expf(-gate))));
        }
        __syncthreads();
    }
    if (mine && n_new > 0 && mode != ML_FROM_STARTS) {
        if (dim == DMAX) {
#pragma unroll
            for (int d = 0; d < DMAX; ++d) sp[(size_t)d * cols] = S[d];
        } else {
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < dim) sp[(size_t)d * cols] = S[d];
        }
    }
    if (wave == 0 && n_new > 0 && mode != ML_FROM_STARTS) {
#pragma unroll
        for (int i = 0; i < QREGS; ++i) {
            const int d = i * WAVE + lane;
            if (d < dim) (sp - v)[(size_t)d * cols + vdim] = nreg[i];
        }
    }
    if (mode == ML_LOCAL && v == 0) chunk_keep[((size_t)b * max_chunks + c) * heads + h] = kept;
}

// Step 2 above: one thread per element of (sequence, head, dim, vdim + 1).  starts[b][c] holds L_c and leaves as S_c.
__global__ void mlstm_starts_kernel(float* __restrict__ starts, const float* __restrict__ chunk_keep, float* __restrict__ state,
                                    const int* __restrict__ seq_slot, const int* __restrict__ seq_new, int chunk, int max_chunks,
                                    int heads, int per_head) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (e >= heads * per_head) return;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const int h = e / per_head;
    float* st = state + (size_t)seq_slot[b] * heads * per_head + e;
    float s = *st;
    for (int c = 0; c * chunk < n_new; ++c) {
        float* at = starts + ((size_t)b * max_chunks + c) * heads * per_head + e;
        const float local = *at;
        *at = s;
        s = fmaf(chunk_keep[((size_t)b * max_chunks + c) * heads + h], s, local);
    }
    *st = s;
}

template <typename T>
static void mlstm_launch(hipStream_t stream, dim3 grid, int threads, int mode, int chunk, int max_chunks, float* starts, float* chunk_keep,
                         const T* rows, int row_stride, int v_off, int g_off, const float* qk, const float4* coef, const float* norm_w,
                         float eps, float* state, const int* seq_slot, const int* seq_new, const int* cu_new, int heads, int dim, int vdim,
                         T* out) {
#define ML_CASE(D) { if (threads <= 256) mlstm_kernel<T, D, 256><<<grid, threads, 0, stream>>>(mode, chunk, max_chunks, starts, chunk_keep, rows, \
            row_stride, v_off, g_off, qk, coef, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, out); \
        else mlstm_kernel<T, D, 1024><<<grid, threads, 0, stream>>>(mode, chunk, max_chunks, starts, chunk_keep, rows, \
            row_stride, v_off, g_off, qk, coef, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, out); }
    if (dim <= 32) ML_CASE(32)
    else if (dim <= 64) ML_CASE(64)
    else if (dim <= 128) ML_CASE(128)
    else ML_CASE(256)
#undef ML_CASE
}

PALM_API int palm_mlstm_pad(int dim) { return dim <= 32 ? 32 : dim <= 64 ? 64 : dim <= 128 ? 128 : 256; }

// rows [n, row_stride]: q | k | v | gate at their offsets; gates float32 [n, 2 heads] with gate_bias float32 [2 heads] or null;
// state float32 [slots, heads, dim, vdim + 1], m_state float32 [slots, heads]; norm_w float32 [heads * vdim]; out [n, heads * vdim].
// Room: qk n * heads * 2 * pad floats, coef n * heads * 4 floats; with chunks (chunk > 0), max_chunks = ceil(max_new / chunk):
// starts n_seqs * max_chunks * heads * dim * (vdim + 1) floats and chunk_keep n_seqs * max_chunks * heads floats.
PALM_API int palm_mlstm(hipStream_t stream, const void* rows, int dtype, int row_stride, int q_off, int k_off, int v_off, int g_off,
                        const float* gates, const float* gate_bias, float cap, float q_scale, const float* norm_w, float eps, float* state,
                        float* m_state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs, int heads, int dim,
                        int vdim, void* out, int max_new, int chunk, float* starts, float* chunk_keep, int n_tokens, float* qk, float* coef) {
    PALM_CHECK(n_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0, "mlstm: seqs=%d heads=%d dim=%d vdim=%d", n_seqs, heads, dim, vdim);
    PALM_CHECK(dim <= 256, "mlstm: a key size of %d exceeds 256", dim);
    PALM_CHECK(vdim <= 1024, "mlstm: a value size of %d exceeds 1024", vdim);
    PALM_CHECK(cap > 0.f, "mlstm: the gates' cap %f must be positive", cap);
    PALM_CHECK(chunk >= 0 && (chunk == 0 || (starts && chunk_keep && max_new > 0)), "mlstm: chunks of %d tokens need their starting states", chunk);
    PALM_CHECK(n_tokens == 0 || (qk && coef && gates && norm_w && state && m_state && out), "mlstm: rows, factors and state need their room");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    const int max_chunks = chunk > 0 ? (max_new + chunk - 1) / chunk : 1;
    PALM_CHECK(heads <= 65535 && (long long)n_seqs * max_chunks <= 65535, "mlstm: %d heads / %d sequences x %d chunks are more than one launch takes",
               heads, n_seqs, max_chunks);
    const int threads = (vdim + WAVE - 1) / WAVE * WAVE;
    dim3 grid(heads, n_seqs * max_chunks);
    const int pad = palm_mlstm_pad(dim);
    const long long qk_threads = (long long)n_tokens * heads * pad;
    mlstm_gates_kernel<<<dim3(heads, n_seqs), WAVE, 0, stream>>>(gates, gate_bias, cap, m_state, seq_slot, seq_new, cu_new, heads, (float4*)coef);
    PALM_DTYPE_SWITCH(dtype, T, {
        mlstm_qk_kernel<T><<<(unsigned)((qk_threads + 255) / 256), 256, 0, stream>>>((const T*)rows, row_stride, q_off, k_off, q_scale, n_tokens,
                                                                                    heads, dim, pad, qk);
        if (chunk == 0) {
            mlstm_launch<T>(stream, grid, threads, ML_WHOLE, 1 << 30, 1, nullptr, nullptr, (const T*)rows, row_stride, v_off, g_off, qk,
                            (const float4*)coef, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out);
        } else {
            mlstm_launch<T>(stream, grid, threads, ML_LOCAL, chunk, max_chunks, starts, chunk_keep, (const T*)rows, row_stride, v_off, g_off, qk,
                            (const float4*)coef, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out);
            const int elems = heads * dim * (vdim + 1);
            mlstm_starts_kernel<<<dim3((elems + 255) / 256, n_seqs), 256, 0, stream>>>(starts, chunk_keep, state, seq_slot, seq_new, chunk,
                                                                                     max_chunks, heads, dim * (vdim + 1));
            mlstm_launch<T>(stream, grid, threads, ML_FROM_STARTS, chunk, max_chunks, starts, chunk_keep, (const T*)rows, row_stride, v_off, g_off,
                            qk, (const float4*)coef, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out);
        }
    });
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
