// Causal grouped-query softmax attention over the paged cache with the options that the plain attention kernels do not
// have: a key size and a value size of their own, an RMS norm over the whole q projection and the whole k projection
// (or per head, or none), biases on q, k and v, a rotation of the first `rot` dimensions of each head, a sliding
// window, a sink (a key of a fixed score without a value: it only adds exp(score) to the softmax's denominator), and an
// elementwise sigmoid gate on the heads' outputs (or one gate value for each head).  The sink's score is one number for
// all heads or a learned one for each.  Between the bias and the norm q, k and v may go through a short causal convolution
// over time, a channel at a time: y_t = sum_j w[c][j] u_(t - taps + 1 + j) with zeros before the sequence's start; the last
// taps - 1 inputs u of each sequence are kept as state.  The rotation pairs dimension i with i + rot/2, or 2i with 2i + 1.
//
//   p_j = exp(s_j) / (exp(sink) + sum_i exp(s_i)),   s_j = scale * q . k_j,   max(0, pos - window + 1) <= j <= pos
//   out = (sum_j p_j v_j) * sigmoid(gate)
//
// K is [pages, kv_heads, 64, dim]; V is kept transposed, [pages, kv_heads, vdim, 64].
//
// This file: the pass that norms and rotates q and k and writes the step's keys and values to their pages, and the
// exact kernel (32-bit arithmetic), which serves the float32 mode, single tokens, and whatever the matrix-core kernel
// does not take.  One block of four waves per (query, group of up to eight query heads that share a key/value head,
// slice of the key range): a key or value is read once for all those heads.  A wave takes every fourth page of the
// slice; in a page each lane scores one key for all heads and owns a few value columns (the weights reach all lanes
// through LDS), the wave keeps a running (max, sum, output) for each head, and the four waves' partial results are
// merged at the end.  With one slice the block then gates and writes the
// output; with more (a decode step: few queries over long ranges) it leaves its partial result in a workspace for
// the merging kernel.
#include "common.h"

constexpr int SK_WAVES = 4;
constexpr int SK_MAX_DIM = 256;            // of keys and of values
constexpr int SK_VACC = SK_MAX_DIM / WAVE;
constexpr int SK_MAX_GROUP = 8;            // query heads a block takes at once

enum SinkNorm : int { SK_NORM_NONE = 0, SK_NORM_PROJECTION = 1, SK_NORM_HEAD = 2 };

// ---- q, k, v of the step's tokens ---------------------------------------------------------------------------
// One block per token.  The projection-wide sums of squares are made by the whole block; then a wave takes a head
// (of q or of k) at a time: norm, weight, rotation, and q goes to q_out, k to its page.
template <typename T>
__global__ __launch_bounds__(1024) void sink_qkv_store_kernel(
    const T* __restrict__ rows, int stride, int q_off, int k_off, int v_off, const float* __restrict__ bias,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ block_table, int max_pages,
    const int* __restrict__ tok_slot, const int* __restrict__ positions, int norm_mode, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
    int heads, int kv_heads, int dim, int vdim, int write_cache, int pairing,
    const float* __restrict__ conv_w, int taps, float* __restrict__ conv_state, int conv_channels, int fuse_state) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const T* row = rows + t * stride;
    const int q_size = heads * dim, k_size = kv_heads * dim;
    const float* q_b = bias, * k_b = bias ? bias + q_size : nullptr, * v_b = bias ? bias + q_size + k_size : nullptr;
    const int pos = positions[t];
    const int page = write_cache ? block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS] : 0;
    const int at = pos % PAGE_TOKENS;
    // The convolution's inputs: of the rows right before this one, `before` belong to the same sequence (a sequence's rows lie
    // together); what lies further back comes from the sequence's state, oldest first, zero for a sequence that has just begun.
    int before = 0;
    const float* st = nullptr;
    if (taps > 1) {
        const int slot = tok_slot[t];
        while (before < taps - 1 && t > (size_t)before && tok_slot[t - before - 1] == slot) ++before;
        st = conv_state + (size_t)slot * (taps - 1) * conv_channels;
    }
    // column `col` of the rows, which is channel `ch` of q | k | v, with its bias, through the convolution
    auto value = [&](int col, int ch, const float* b) {
        const float bias_c = b ? *b : 0.f;
        if (taps <= 1) return (to_float(row[col]) + bias_c) * (taps == 1 ? conv_w[ch] : 1.f);      // (one tap: a factor a channel)
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int back = taps - 1 - j;
            const float u = back <= before ? to_float(rows[(t - back) * stride + col]) + bias_c
                                           : st[(size_t)(taps - 1 - (back - before)) * conv_channels + ch];
            acc = fmaf(conv_w[(size_t)ch * taps + j], u, acc);
        }
        return acc;
    };
    float inv_q = 1.f, inv_k = 1.f;
    if (norm_mode == SK_NORM_PROJECTION) {
        float sq = 0.f, sk = 0.f;
        for (int i = threadIdx.x; i < q_size; i += blockDim.x) { const float v = value(q_off + i, i, q_b ? q_b + i : nullptr); sq += v * v; }
        for (int i = threadIdx.x; i < k_size; i += blockDim.x) { const float v = value(k_off + i, q_size + i, k_b ? k_b + i : nullptr); sk += v * v; }
        sq = block_sum(sq, scratch);
        sk = block_sum(sk, scratch);
        inv_q = 1.0f / sqrtf(sq / (float)q_size + eps);
        inv_k = 1.0f / sqrtf(sk / (float)k_size + eps);
    }
    const int half = rot / 2;
    for (int r = wave; r < heads + kv_heads; r += n_waves) {
        const bool is_q = r < heads;
        if (!is_q && !write_cache) continue;
        const int hh = is_q ? r : r - heads;
        const int col0 = (is_q ? q_off : k_off) + hh * dim, ch0 = (is_q ? 0 : q_size) + hh * dim;
        const float* b = is_q ? (q_b ? q_b + (size_t)hh * dim : nullptr) : (k_b ? k_b + (size_t)hh * dim : nullptr);
        float inv = is_q ? inv_q : inv_k;
        const float* w = nullptr;
        if (norm_mode == SK_NORM_PROJECTION) w = (is_q ? q_w : k_w) + (size_t)hh * dim;
        if (norm_mode == SK_NORM_HEAD) {
            w = is_q ? q_w : k_w;
            float ss = 0.f;
            for (int d = lane; d < dim; d += WAVE) { const float v = value(col0 + d, ch0 + d, b ? b + d : nullptr); ss += v * v; }
            inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
        }
        T* dst = is_q ? q_out + (t * heads + hh) * dim
                      : k_cache + (((size_t)page * kv_heads + hh) * PAGE_TOKENS + at) * dim;
        auto normed = [&](int d) {
            const float v = value(col0 + d, ch0 + d, b ? b + d : nullptr) * inv;
            return w ? v * w[d] : v;
        };
        for (int d = lane; d < dim; d += WAVE) {
            float v = normed(d);
            if (d < rot) {
                // pairs (i, i + rot/2), or neighbours (2i, 2i + 1)
                const bool first = pairing == 1 ? (d & 1) == 0 : d < half;
                const int i = pairing == 1 ? d >> 1 : (d < half ? d : d - half);
                const int partner = pairing == 1 ? d ^ 1 : (d < half ? d + half : d - half);
                const float c = cos_t[t * half + i], sn = sin_t[t * half + i];
                const float pv = normed(partner);
                // the pair (u, w) becomes (u c - w s, w c + u s)
                v = first ? v * c - pv * sn : v * c + pv * sn;
            }
            dst[d] = from_float<T>(v);
        }
    }
    if (write_cache) {
        for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x)
            v_cache[((size_t)page * kv_heads * vdim + i) * PAGE_TOKENS + at] = from_float<T>(value(v_off + i, q_size + k_size + i, v_b ? v_b + i : nullptr));
    }
    // Every sequence of the step brings one token: this block is the only one that touches its sequence's state, and moves
    // it on by its token once all the block's reads of the old state are done.
    if (fuse_state && taps > 1) {
        __syncthreads();
        float* stw = conv_state + (size_t)tok_slot[t] * (taps - 1) * conv_channels;
        for (int c = threadIdx.x; c < conv_channels; c += blockDim.x) {
            const int col = c < q_size ? q_off + c : c < q_size + k_size ? k_off + (c - q_size) : v_off + (c - q_size - k_size);
            const float cur = to_float(row[col]) + (bias ? bias[c] : 0.f);
            for (int j = 0; j + 2 < taps; ++j) stw[(size_t)j * conv_channels + c] = stw[(size_t)(j + 1) * conv_channels + c];
            stw[(size_t)(taps - 2) * conv_channels + c] = cur;
        }
    }
}

// After the pass above has read the old state: the last taps - 1 inputs (projection plus bias) of each sequence, old ones
// moved up.  One thread per (channel, sequence); a thread reads all it keeps before it writes.
constexpr int SK_MAX_TAPS = 16;

template <typename T>
__global__ void sink_conv_state_kernel(const T* __restrict__ rows, int stride, int q_off, int k_off, int v_off, int q_size, int k_size,
                                       const float* __restrict__ bias, float* __restrict__ conv_state, const int* __restrict__ seq_slot,
                                       const int* __restrict__ seq_new, const int* __restrict__ cu_new, int channels, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= channels) return;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const int col = c < q_size ? q_off + c : c < q_size + k_size ? k_off + (c - q_size) : v_off + (c - q_size - k_size);
    const float bias_c = bias ? bias[c] : 0.f;
    const size_t row0 = (size_t)cu_new[b];
    float* st = conv_state + (size_t)seq_slot[b] * (taps - 1) * channels;
    float keep[SK_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < SK_MAX_TAPS; ++j) {
        if (j < taps - 1) {
            const int at = n_new - (taps - 1) + j;
            keep[j] = at >= 0 ? to_float(rows[(row0 + at) * stride + col]) + bias_c : st[(size_t)(taps - 1 + at) * channels + c];
        }
    }
#pragma unroll
    for (int j = 0; j < SK_MAX_TAPS; ++j)
        if (j < taps - 1) st[(size_t)j * channels + c] = keep[j];
}

PALM_API int palm_sink_qkv_store(hipStream_t stream, const void* rows, int dtype, int stride, int q_off, int k_off, int v_off,
                                 const float* bias, void* q_out, void* k_cache, void* v_cache, const int* block_table, int max_pages,
                                 const int* tok_slot, const int* positions, int norm_mode, const float* q_w, const float* k_w, float eps,
                                 const float* cos_t, const float* sin_t, int rot, int n_tokens, int heads, int kv_heads, int dim, int vdim,
                                 int write_cache, int pairing, const float* conv_w, int taps, float* conv_state, const int* seq_slot,
                                 const int* seq_new, const int* cu_new, int n_seqs) {
    PALM_CHECK(n_tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "sink_qkv_store: tokens=%d heads=%d kv=%d dim=%d vdim=%d",
               n_tokens, heads, kv_heads, dim, vdim);
    PALM_CHECK(norm_mode >= SK_NORM_NONE && norm_mode <= SK_NORM_HEAD, "sink_qkv_store: norm mode %d", norm_mode);
    PALM_CHECK(norm_mode == SK_NORM_NONE || (q_w && k_w), "sink_qkv_store: a norm needs its weights");
    PALM_CHECK(rot >= 0 && rot <= dim && rot % 2 == 0, "sink_qkv_store: %d rotated dimensions of %d", rot, dim);
    PALM_CHECK(rot == 0 || (cos_t && sin_t), "sink_qkv_store: a rotation needs its cos and sin rows");
    PALM_CHECK(!write_cache || (k_cache && v_cache && block_table && tok_slot && max_pages > 0), "sink_qkv_store: writing needs cache, pages and slots");
    PALM_CHECK(pairing == 0 || pairing == 1, "sink_qkv_store: pairing %d is neither halves (0) nor neighbours (1)", pairing);
    PALM_CHECK(taps >= 0 && taps <= SK_MAX_TAPS, "sink_qkv_store: %d taps (at most %d)", taps, SK_MAX_TAPS);
    PALM_CHECK(taps <= 1 || (conv_w && conv_state && tok_slot && seq_slot && seq_new && cu_new && n_seqs > 0 && n_seqs <= 65535),
               "sink_qkv_store: a convolution needs its weights, its state and the step's sequences");
    if (n_tokens == 0) return 0;
    // the convolution's channels: q, and k and v if this layer makes them
    const int conv_channels = heads * dim + (write_cache ? kv_heads * (dim + vdim) : 0);
    // one token a sequence (a decode step): the pass moves the state on itself; else a second launch does, after all reads
    const int fuse_state = taps > 1 && n_tokens == n_seqs;
    // a wave takes a head at a time: for few tokens (a decode step) as many waves as there are heads of q and k, within a
    // block's sixteen; many tokens fill the chip anyway
    const int threads = n_tokens >= 256 ? 256 : min(1024, max(256, WAVE * (heads + kv_heads)));
    PALM_DTYPE_SWITCH(dtype, T,
        sink_qkv_store_kernel<T><<<n_tokens, threads, 0, stream>>>((const T*)rows, stride, q_off, k_off, v_off, bias, (T*)q_out, (T*)k_cache,
                                                              (T*)v_cache, block_table, max_pages, tok_slot, positions, norm_mode, q_w, k_w,
                                                              eps, cos_t, sin_t, rot, heads, kv_heads, dim, vdim, write_cache, pairing,
                                                              conv_w, taps, conv_state, conv_channels, fuse_state);
        if (taps > 1 && !fuse_state)
            sink_conv_state_kernel<T><<<dim3((conv_channels + 255) / 256, n_seqs), 256, 0, stream>>>(
                (const T*)rows, stride, q_off, k_off, v_off, heads * dim, kv_heads * dim, bias, conv_state, seq_slot, seq_new, cu_new,
                conv_channels, taps));
    PALM_LAUNCHED();
    return 0;
}

// ---- the exact kernel -------------------------------------------------------------------------------------
// 16 bytes of a row at a time where the sizes allow.
template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    __device__ static void unpack(const uint4 v, float (&o)[4]) {
        o[0] = __builtin_bit_cast(float, v.x); o[1] = __builtin_bit_cast(float, v.y);
        o[2] = __builtin_bit_cast(float, v.z); o[3] = __builtin_bit_cast(float, v.w);
    }
    __device__ static void load(const float* p, float (&o)[4]) { unpack(*reinterpret_cast<const uint4*>(p), o); }
};
template <> struct Vec16<bf16_t> {
    static constexpr int N = 8;
    __device__ static void load(const bf16_t* p, float (&o)[8]) { unpack(*reinterpret_cast<const uint4*>(p), o); }
    __device__ static void unpack(const uint4 v, float (&o)[8]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __builtin_bit_cast(float, w[i] << 16);
            o[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
        }
    }
};

// Workspace of a (token, head, slice): m, l, then vdim sums.  NV: value columns a lane (the value size over 64, rounded up),
// a number of the build so that the innermost loops hold no test.
template <typename T, int MAXQ, int NV>
__global__ __launch_bounds__(SK_WAVES * WAVE) void sink_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table,
    int max_pages, const int* __restrict__ seq_slot, const int* __restrict__ seq_start, const int* __restrict__ seq_new,
    const int* __restrict__ cu_new, int heads, int kv_heads, int dim, int vdim, float scale, int window, int has_sink,
    float sink_score, const float* __restrict__ sink_scores, const T* __restrict__ gate, int gate_stride, int gate_per_head, int n_slices,
    float* __restrict__ work, T* __restrict__ out) {
    __shared__ float q_s[MAXQ][SK_MAX_DIM];
    __shared__ float m_s[SK_WAVES][MAXQ], l_s[SK_WAVES][MAXQ];
    __shared__ float acc_s[SK_WAVES][MAXQ][SK_MAX_DIM];
    __shared__ float p_s[SK_WAVES][MAXQ][PAGE_TOKENS];           // a wave's weights of the page at hand, for all its lanes to read

    const int per_kv = heads / kv_heads;
    const int chunks = (per_kv + MAXQ - 1) / MAXQ;                 // a group of more than MAXQ heads goes through in several blocks
    const int qi = blockIdx.x, g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int b = blockIdx.z / n_slices, slice = blockIdx.z % n_slices;
    if (qi >= seq_new[b]) return;
    const int h0 = g * per_kv + chunk * MAXQ;
    const int nq = min(MAXQ, per_kv - chunk * MAXQ);
    const int t = cu_new[b] + qi;
    const int pos = seq_start[b] + qi;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    for (int i = threadIdx.x; i < MAXQ * dim; i += blockDim.x) {
        const int qh = i / dim, d = i % dim;
        q_s[qh][d] = qh < nq ? to_float(q[((size_t)t * heads + h0 + qh) * dim + d]) * scale : 0.f;
    }
    __syncthreads();

    float m[MAXQ], l[MAXQ], acc[MAXQ][NV];
#pragma unroll
    for (int qh = 0; qh < MAXQ; ++qh) {
        const bool sink_here = has_sink && slice == 0 && wave == 0;
        // one score for all heads, or a learned one for each
        m[qh] = sink_here ? (sink_scores ? sink_scores[min(h0 + qh, heads - 1)] : sink_score) : -INFINITY;
        l[qh] = sink_here && lane == 0 ? 1.f : 0.f;              // (a lane's part of the running sum)
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[qh][i] = 0.f;
    }

    // this slice's pages
    const int p_lo = lo / PAGE_TOKENS, p_hi = pos / PAGE_TOKENS;
    const int per_slice = (p_hi - p_lo + n_slices) / n_slices;
    const int s_lo = p_lo + slice * per_slice, s_hi = min(p_hi, s_lo + per_slice - 1);
    constexpr int VN = Vec16<T>::N;
    const bool k_vec = dim % VN == 0;
    const bool k_full = dim % (4 * VN) == 0, v_full = vdim % WAVE == 0;

    for (int pg = s_lo + wave; pg <= s_hi; pg += SK_WAVES) {
        const int page = pages[pg];
        const T* kp = k_cache + ((size_t)page * kv_heads + g) * PAGE_TOKENS * dim;
        const T* vp = v_cache + ((size_t)page * kv_heads + g) * (size_t)vdim * PAGE_TOKENS;
        const int j = pg * PAGE_TOKENS + lane;
        const bool seen = j >= lo && j <= pos;
        float s[MAXQ];
#pragma unroll
        for (int qh = 0; qh < MAXQ; ++qh) s[qh] = 0.f;
        const T* kr = kp + (size_t)lane * dim;
        // 2-byte elements: the lane's rows of the transposed value page (128 bytes each) are all asked for here, before
        // the scores are made, so that they arrive while the softmax is at work
        constexpr bool V_AHEAD = sizeof(T) == 2;
        uint4 vraw[V_AHEAD ? NV : 1][V_AHEAD ? PAGE_TOKENS / VN : 1];
        if constexpr (V_AHEAD) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                // (a value size of whole waves, the usual case, needs no clamp: plain strides make the cheapest addresses)
                const T* vr = vp + (size_t)(v_full ? lane + i * WAVE : min(lane + i * WAVE, vdim - 1)) * PAGE_TOKENS;
#pragma unroll
                for (int c8 = 0; c8 < PAGE_TOKENS / VN; ++c8) vraw[i][c8] = *reinterpret_cast<const uint4*>(vr + c8 * VN);
            }
        }
        if (k_full) {
            // four reads of 16 bytes are under way together
            for (int d0 = 0; d0 < dim; d0 += 4 * VN) {
                uint4 raw[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) raw[u] = *reinterpret_cast<const uint4*>(kr + d0 + u * VN);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    float kv[VN];
                    Vec16<T>::unpack(raw[u], kv);
#pragma unroll
                    for (int e = 0; e < VN; ++e)
#pragma unroll
                        for (int qh = 0; qh < MAXQ; ++qh) s[qh] = fmaf(q_s[qh][d0 + u * VN + e], kv[e], s[qh]);
                }
            }
        } else if (k_vec) {
            // (the last reads of a row that is no multiple of four reads repeat its end and are not used)
            for (int d0 = 0; d0 < dim; d0 += 4 * VN) {
                uint4 raw[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) raw[u] = *reinterpret_cast<const uint4*>(kr + min(d0 + u * VN, dim - VN));
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (d0 + u * VN >= dim) break;
                    float kv[VN];
                    Vec16<T>::unpack(raw[u], kv);
#pragma unroll
                    for (int e = 0; e < VN; ++e)
#pragma unroll
                        for (int qh = 0; qh < MAXQ; ++qh) s[qh] = fmaf(q_s[qh][d0 + u * VN + e], kv[e], s[qh]);
                }
            }
        } else {
            for (int d = 0; d < dim; ++d) {
                const float kd = to_float(kr[d]);
#pragma unroll
                for (int qh = 0; qh < MAXQ; ++qh) s[qh] = fmaf(q_s[qh][d], kd, s[qh]);
            }
        }
        // the page's maxima of all heads together: every step's exchanges between lanes are under way at once
        float p[MAXQ], top[MAXQ];
#pragma unroll
        for (int qh = 0; qh < MAXQ; ++qh) top[qh] = s[qh] = seen ? s[qh] : -INFINITY;
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) {
            float other[MAXQ];
#pragma unroll
            for (int qh = 0; qh < MAXQ; ++qh) other[qh] = __shfl_xor(top[qh], off, WAVE);
#pragma unroll
            for (int qh = 0; qh < MAXQ; ++qh) top[qh] = fmaxf(top[qh], other[qh]);
        }
#pragma unroll
        for (int qh = 0; qh < MAXQ; ++qh) {
            const float m_new = fmaxf(m[qh], top[qh]);            // every page of the range holds a key that is seen
            const float alpha = expf(m[qh] - m_new);              // m = -inf at the first page: exp(-inf) = 0
            p[qh] = expf(s[qh] - m_new);                          // a key that is not seen: exp(-inf) = 0
            l[qh] = l[qh] * alpha + p[qh];                        // this lane's part of the sum; the lanes are added at the end
            m[qh] = m_new;
#pragma unroll
            for (int i = 0; i < NV; ++i) acc[qh][i] *= alpha;
        }
        // A lane holds the weight of its key; every lane needs every key's.  They go through LDS (all lanes read one
        // address: one pass), four keys a read, which costs far less than handing them out lane by lane as scalars.
        // The wave's own reads follow its own writes in order; the fences keep the compiler from moving them.
#pragma unroll
        for (int qh = 0; qh < MAXQ; ++qh) p_s[wave][qh][lane] = p[qh];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // values: lane c owns columns c, c + 64, ..; its rows of the transposed page are read 16 bytes at a time
        const int j_first = max(lo, pg * PAGE_TOKENS) - pg * PAGE_TOKENS;
        const int j_last = min(pos, pg * PAGE_TOKENS + PAGE_TOKENS - 1) - pg * PAGE_TOKENS;
        if constexpr (V_AHEAD) {
#pragma unroll
            for (int c8 = 0; c8 < PAGE_TOKENS / VN; ++c8) {
                const int j0 = c8 * VN;
                if (j0 + VN - 1 < j_first || j0 > j_last) continue;       // (the same in every lane)
                float vv[NV][VN];
#pragma unroll
                for (int i = 0; i < NV; ++i) Vec16<T>::unpack(vraw[i][c8], vv[i]);
#pragma unroll
                for (int qh = 0; qh < MAXQ; ++qh) {
#pragma unroll
                    for (int e = 0; e < VN; ++e) {
                        const float pj = p_s[wave][qh][j0 + e];
#pragma unroll
                        for (int i = 0; i < NV; ++i) acc[qh][i] = fmaf(pj, vv[i][e], acc[qh][i]);
                    }
                }
            }
        } else
        for (int j0 = j_first / VN * VN; j0 <= j_last; j0 += VN) {
            float vv[NV][VN];
#pragma unroll
            for (int i = 0; i < NV; ++i) Vec16<T>::load(vp + (size_t)min(lane + i * WAVE, vdim - 1) * PAGE_TOKENS + j0, vv[i]);
#pragma unroll
            for (int qh = 0; qh < MAXQ; ++qh) {
#pragma unroll
                for (int e = 0; e < VN; ++e) {
                    const float pj = p_s[wave][qh][j0 + e];       // zero for a key that is not seen
#pragma unroll
                    for (int i = 0; i < NV; ++i) acc[qh][i] = fmaf(pj, vv[i][e], acc[qh][i]);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // (the next page's weights are written after these reads)
        __builtin_amdgcn_wave_barrier();
    }

#pragma unroll
    for (int qh = 0; qh < MAXQ; ++qh) {
        const float l_wave = wave_sum(l[qh]);
        if (lane == 0) { m_s[wave][qh] = m[qh]; l_s[wave][qh] = l_wave; }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane + i * WAVE;
            if (c < vdim) acc_s[wave][qh][c] = acc[qh][i];
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nq * vdim; i += blockDim.x) {
        const int qh = i / vdim, c = i % vdim, h = h0 + qh;
        float m_all = -INFINITY;
        for (int w = 0; w < SK_WAVES; ++w) m_all = fmaxf(m_all, m_s[w][qh]);
        float l_all = 0.f, o = 0.f;
        for (int w = 0; w < SK_WAVES; ++w) {
            const float f = m_s[w][qh] == -INFINITY ? 0.f : expf(m_s[w][qh] - m_all);
            l_all += l_s[w][qh] * f;
            o += acc_s[w][qh][c] * f;
        }
        if (n_slices == 1) {
            float r = o / l_all;
            if (gate) { const float gt = to_float(gate[(size_t)t * gate_stride + (gate_per_head ? h : (size_t)h * vdim + c)]); r *= 1.0f / (1.0f + expf(-gt)); }
            out[((size_t)t * heads + h) * vdim + c] = from_float<T>(r);
        } else {
            float* wk = work + (((size_t)t * heads + h) * n_slices + slice) * (vdim + 2);
            if (c == 0) { wk[0] = m_all; wk[1] = l_all; }
            wk[2 + c] = o;
        }
    }
}

// The slices of a (token, head) merged, gated and written: one wave.  The slices' maxima and sums are read a slice a lane
// (all reads under way at once), their weights wait in LDS, and the columns' sums run over the slices four reads at a time.
constexpr int SK_MAX_SLICES = 1024;

template <typename T>
__global__ __launch_bounds__(WAVE) void sink_attention_merge_kernel(const float* __restrict__ work, int n_slices, int heads, int vdim,
                                                                    const T* __restrict__ gate, int gate_stride, int gate_per_head,
                                                                    T* __restrict__ out) {
    __shared__ float w_s[SK_MAX_SLICES];
    const size_t t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const size_t stride = (size_t)(vdim + 2);
    const float* wk = work + ((t * heads + h) * n_slices) * stride;
    float m_loc = -INFINITY;
    for (int s = lane; s < n_slices; s += WAVE) m_loc = fmaxf(m_loc, wk[s * stride]);
    const float m_all = wave_max(m_loc);
    float l_loc = 0.f;
    for (int s = lane; s < n_slices; s += WAVE) {
        const float ms = wk[s * stride];
        const float w = ms == -INFINITY ? 0.f : expf(ms - m_all);
        w_s[s] = w;
        l_loc = fmaf(wk[s * stride + 1], w, l_loc);
    }
    const float l_all = wave_sum(l_loc);
    __syncthreads();
    for (int c = lane; c < vdim; c += WAVE) {
        const float* col = wk + 2 + c;
        float o = 0.f;
        int s = 0;
        for (; s + 4 <= n_slices; s += 4) {
            const float a0 = col[(s + 0) * stride], a1 = col[(s + 1) * stride], a2 = col[(s + 2) * stride], a3 = col[(s + 3) * stride];
            o = fmaf(a0, w_s[s], o); o = fmaf(a1, w_s[s + 1], o); o = fmaf(a2, w_s[s + 2], o); o = fmaf(a3, w_s[s + 3], o);
        }
        for (; s < n_slices; ++s) o = fmaf(col[s * stride], w_s[s], o);
        float r = o / l_all;
        if (gate) { const float gt = to_float(gate[t * gate_stride + (gate_per_head ? h : (size_t)h * vdim + c)]); r *= 1.0f / (1.0f + expf(-gt)); }
        out[(t * heads + h) * vdim + c] = from_float<T>(r);
    }
}

// q [n, heads, dim]; gate: null, or the first gate value of token 0 (rows `gate_stride` elements apart, heads * vdim
// values a row, or with gate_per_head one value for each head); sink_scores: null, or a score for each head; work: room for n_tokens * heads * n_slices * (vdim + 2) floats if n_slices > 1; out [n, heads * vdim].
PALM_API int palm_sink_attention(hipStream_t stream, const void* q, int dtype, const void* k_cache, const void* v_cache,
                                 const int* block_table, int max_pages, const int* seq_slot, const int* seq_start, const int* seq_new,
                                 const int* cu_new, int n_seqs, int max_new, int n_tokens, int heads, int kv_heads, int dim, int vdim,
                                 float scale, int window, int has_sink, float sink_score, const float* sink_scores, const void* gate,
                                 int gate_stride, int gate_per_head, int n_slices, float* work, void* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0,
               "sink_attention: seqs=%d max_new=%d heads=%d kv=%d dim=%d vdim=%d", n_seqs, max_new, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "sink_attention: %d heads are not a multiple of %d kv heads", heads, kv_heads);
    PALM_CHECK(dim <= SK_MAX_DIM && vdim <= SK_MAX_DIM, "sink_attention: key size %d / value size %d exceed %d", dim, vdim, SK_MAX_DIM);
    PALM_CHECK(window >= 0 && max_pages > 0, "sink_attention: window %d, max_pages %d", window, max_pages);
    PALM_CHECK(n_slices >= 1 && n_slices <= SK_MAX_SLICES && (n_slices == 1 || work), "sink_attention: %d slices (at most %d) need a workspace",
               n_slices, SK_MAX_SLICES);
    if (n_seqs == 0 || max_new == 0 || n_tokens == 0) return 0;
    const int per_kv = heads / kv_heads;
    const int maxq = per_kv >= 8 ? 8 : per_kv > 2 ? 4 : per_kv;
    const int chunks = (per_kv + maxq - 1) / maxq;
    PALM_CHECK(kv_heads * chunks <= 65535 && (long long)n_seqs * n_slices <= 65535,
               "sink_attention: %d kv heads / %d sequences x %d slices are more than one launch takes", kv_heads, n_seqs, n_slices);
    dim3 grid(max_new, kv_heads * chunks, n_seqs * n_slices);
    const int nv = (vdim + WAVE - 1) / WAVE;
#define SK_CASE_V(Q, V) sink_attention_kernel<T, Q, V><<<grid, SK_WAVES * WAVE, 0, stream>>>((const T*)q, (const T*)k_cache, (const T*)v_cache, \
        block_table, max_pages, seq_slot, seq_start, seq_new, cu_new, heads, kv_heads, dim, vdim, scale, window, has_sink, sink_score, \
        sink_scores, (const T*)gate, gate_stride, gate_per_head, n_slices, work, (T*)out)
#define SK_CASE(Q) { if (nv == 1) SK_CASE_V(Q, 1); else if (nv == 2) SK_CASE_V(Q, 2); else if (nv == 3) SK_CASE_V(Q, 3); else SK_CASE_V(Q, 4); }
    PALM_DTYPE_SWITCH(dtype, T, {
        if (maxq == 1) SK_CASE(1) else if (maxq == 2) SK_CASE(2) else if (maxq == 4) SK_CASE(4) else SK_CASE(8)
        if (n_slices > 1)
            sink_attention_merge_kernel<T><<<dim3(n_tokens, heads), 64, 0, stream>>>(work, n_slices, heads, vdim, (const T*)gate, gate_stride,
                                                                                    gate_per_head, (T*)out);
    });
#undef SK_CASE
#undef SK_CASE_V
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
