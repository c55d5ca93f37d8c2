// Retention: linear attention with one fixed decay per head, no softmax and no denominator.
//
//   S_t = g_h S_(t-1) + k_t v_t^T        S: [dim, vdim] per sequence and head, 32-bit, kept between steps
//   o_t = S_t^T q_t
//   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * silu(gate_t)         (the unit norm is per head)
//
// q and k are rotated first (pairs (i, i + rot/2) of the first `rot` dimensions, cos/sin rows of the tokens'
// positions) and k is multiplied by k_scale after the rotation; rotated values, state and sums are 32-bit.
//
// Two options make this the recurrence of other linear attentions as well: `act` puts q, k and v through silu first
// (q and k before the rotation), and `joined` leaves out the per-head unit norm and the gate: the heads' o_t are then
// written as they are, 32-bit, and a pass of its own norms a token's joined heads together, with a weight, and gates
// them (palm_joined_norm_gate).
//
// A first pass rotates q and k of all the step's tokens into 32-bit rows.  Then one block per (head, sequence), one
// thread per value dimension v: the thread keeps column v of S in registers and walks over the sequence's new
// tokens.  A token's rotated q and k are the same for every thread of the block: each wave reads the two rows once,
// one value a lane, and broadcasts value d to all its lanes as a scalar operand of the multiply-adds (no LDS and no
// barrier in the recurrence); the per-token sums of squares over v are reduced a tile of tokens at a time.  A prompt and a single token run the same code, so a prompt leaves the state that its tokens
// one by one leave.
//
// A long run of new tokens would keep only (heads x sequences) blocks busy, one after the other token.  Such a run is
// cut into chunks of `chunk` tokens, and the recurrence's linearity does the rest in three launches:
//   1. every chunk alone from a zero state: its own sum  L_c = sum_t g^(end - t) k_t v_t^T         (all chunks at once)
//   2. the chunks' starting states, one after the other: S_(c+1) = g^len_c S_c + L_c, S_0 the kept state   (elementwise)
//   3. every chunk from its starting state, now with outputs                                        (all chunks at once)
// The arithmetic of a token is the same in all three; only the order of the 32-bit sums over the past differs.
#include "common.h"

constexpr int RET_TILE = 8;

enum RetentionMode : int { RET_WHOLE = 0, RET_LOCAL = 1, RET_FROM_STARTS = 2 };

__device__ inline float ret_silu(float z) { return z / (1.0f + expf(-z)); }

// q and k of every token and head, rotated (k also scaled), 32-bit: qk[row][head][0 = q, 1 = k][pad], pad >= dim the
// key size that the main kernel is compiled for; the columns beyond dim are zero, so that the main kernel's loops
// over pad need no test (a zero k leaves its row of S zero, a zero q adds nothing).
template <typename T>
__global__ void retention_rotate_kernel(const T* __restrict__ qkvg, int row_stride, int q_off, int k_off,
                                        const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, float k_scale,
                                        int act, int n_tokens, int heads, int dim, int pad, float* __restrict__ qk) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)n_tokens * heads * pad) return;
    const int d = (int)(idx % pad), h = (int)((idx / pad) % heads);
    const size_t row = (size_t)(idx / ((long long)pad * heads));
    float* o = qk + ((row * heads + h) * 2) * pad + d;
    if (d >= dim) { o[0] = 0.f; o[pad] = 0.f; return; }
    const int half = rot / 2;
    const T* qr = qkvg + row * row_stride + q_off + h * dim;
    const T* kr = qkvg + row * row_stride + k_off + h * dim;
    float qv = to_float(qr[d]), kv = to_float(kr[d]);
    if (act) { qv = ret_silu(qv); kv = ret_silu(kv); }
    if (d < rot) {
        const int i = d < half ? d : d - half;
        const float c = cos_t[row * half + i], sn = sin_t[row * half + i];
        const int partner = d < half ? d + half : d - half;
        float qp = to_float(qr[partner]), kp = to_float(kr[partner]);
        if (act) { qp = ret_silu(qp); kp = ret_silu(kp); }
        // the pair (u, w) becomes (u c - w s, w c + u s)
        qv = d < half ? qv * c - qp * sn : qv * c + qp * sn;
        kv = d < half ? kv * c - kp * sn : kv * c + kp * sn;
    }
    o[0] = qv;
    o[pad] = kv * k_scale;
}

// MAXT: the most threads of a block (the value size, rounded up to whole waves): what the compiler may assume when it
// hands out registers.  A thread keeps DMAX values of S; up to 256 threads a block they all stay in registers.
template <typename T, int DMAX, int MAXT>
__global__ __launch_bounds__(MAXT) void retention_kernel(int mode, int chunk, int max_chunks, float* __restrict__ starts, const T* __restrict__ qkvg,
                                 int row_stride, int v_off, int g_off, const float* __restrict__ qk,
                                 const float* __restrict__ decay, float eps,
                                 float* __restrict__ state, const int* __restrict__ seq_slot,
                                 const int* __restrict__ seq_new, const int* __restrict__ cu_new,
                                 int heads, int dim, int vdim, T* __restrict__ out, int act, int joined, float* __restrict__ raw) {
    __shared__ float red[RET_TILE][16];
    __shared__ float o_s[RET_TILE][MAXT];
    constexpr int QREGS = (DMAX + WAVE - 1) / WAVE;
    const int h = blockIdx.x, b = blockIdx.y / max_chunks, c = blockIdx.y % max_chunks;
    const int v = threadIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    // this block's run of tokens: the sequence's new ones, or one chunk of them
    const int seq_tokens = seq_new[b];
    if (c * chunk >= seq_tokens) return;
    const int n_new = mode == RET_WHOLE ? seq_tokens : min(chunk, seq_tokens - c * chunk);
    const int row0 = cu_new[b] + (mode == RET_WHOLE ? 0 : c * chunk);
    const bool mine = v < vdim;
    const float g = decay[h];
    float* sp = mode == RET_WHOLE ? state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim + v
                                  : starts + ((((size_t)b * max_chunks + c) * heads + h) * dim) * vdim + v;

    // the reads are unconditional (of a row and a column that exist) and what does not belong is set to zero after:
    // no branch between them, so that they are all under way at once
    float S[DMAX];
    {
        const float* at = sp - v + min(v, vdim - 1);
        const bool zero = mode == RET_LOCAL || !mine;
        if (dim == DMAX) {                                        // the usual case: every row exists, one stride for all reads
            const size_t stride = (size_t)vdim;
#pragma unroll
            for (int d = 0; d < DMAX; ++d) S[d] = at[d * stride];
            if (zero) {
#pragma unroll
                for (int d = 0; d < DMAX; ++d) S[d] = 0.f;
            }
        } else {
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float s0 = at[(size_t)min(d, dim - 1) * vdim];
                S[d] = (zero || d >= dim) ? 0.f : s0;
            }
        }
    }

    // A token's inputs: the thread's value, and of the token's q and k rows (the same for all threads) one value a
    // lane, which the wave hands to all its lanes as scalars.  The next token's are read while this one's are used.
    const int vc = min(v, vdim - 1);
    auto read_token = [&](int t, float& vv, float (&qv)[QREGS], float (&kv)[QREGS]) {
        const size_t row = (size_t)(row0 + t);
        vv = to_float(qkvg[row * row_stride + v_off + h * vdim + vc]);
        if (act) vv = ret_silu(vv);
        const float* __restrict__ qr = qk + ((row * heads + h) * 2) * DMAX;
#pragma unroll
        for (int c = 0; c < QREGS; ++c) {
            const int at = min(c * WAVE + lane, DMAX - 1);             // (a key size of 32: the upper lanes repeat)
            qv[c] = qr[at];
            kv[c] = qr[DMAX + at];
        }
    };
    float vv, qv[QREGS], kv[QREGS];
    if (n_new > 0) read_token(0, vv, qv, kv);
    for (int t0 = 0; t0 < n_new; t0 += RET_TILE) {
        const int tt = min(RET_TILE, n_new - t0);
        for (int ti = 0; ti < tt; ++ti) {                        // not unrolled: the body is DMAX steps long already
            float vn, qn[QREGS], kn[QREGS];
            read_token(min(t0 + ti + 1, n_new - 1), vn, qn, kn);
            if (!mine) vv = 0.f;
            float acc = 0.f;
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float qd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, qv[d / WAVE]), d % WAVE));
                const float kd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kv[d / WAVE]), d % WAVE));
                S[d] = fmaf(g, S[d], kd * vv);
                acc = fmaf(S[d], qd, acc);
            }
            if (mode != RET_LOCAL && joined) {
                if (mine) raw[(size_t)(row0 + t0 + ti) * ((size_t)heads * vdim) + h * vdim + v] = acc;
            } else if (mode != RET_LOCAL) {
                o_s[ti][v] = acc;
                const float ss = wave_sum(acc * acc);
                if (lane == 0) red[ti][wave] = ss;
            }
            vv = vn;
#pragma unroll
            for (int c = 0; c < QREGS; ++c) { qv[c] = qn[c]; kv[c] = kn[c]; }
        }
        if (mode == RET_LOCAL || joined) continue;
        __syncthreads();
        for (int ti = 0; ti < tt; ++ti) {
            float total = 0.f;
            for (int w = 0; w < n_waves; ++w) total += red[ti][w];
            const float inv = 1.0f / sqrtf(total / (float)vdim + eps);
            const size_t row = (size_t)(row0 + t0 + ti);
            const float gate = to_float(qkvg[row * row_stride + g_off + h * vdim + vc]);
            if (mine) out[row * ((size_t)heads * vdim) + h * vdim + v] = from_float<T>(o_s[ti][v] * inv * (gate / (1.0f + expf(-gate))));
        }
        __syncthreads();
    }
    if (mine && n_new > 0 && mode != RET_FROM_STARTS) {
        if (dim == DMAX) {
#pragma unroll
            for (int d = 0; d < DMAX; ++d) sp[(size_t)d * vdim] = S[d];
        } else {
#pragma unroll
            for (int d = 0; d < DMAX; ++d)
                if (d < dim) sp[(size_t)d * vdim] = S[d];
        }
    }
}

// Step 2 above: one thread per element of (sequence, head, dim, vdim).  starts[b][c] holds L_c and leaves as S_c.
__global__ void retention_starts_kernel(float* __restrict__ starts, float* __restrict__ state, const float* __restrict__ decay,
                                        const int* __restrict__ seq_slot, const int* __restrict__ seq_new, int chunk,
                                        int max_chunks, int heads, int per_head) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (e >= heads * per_head) return;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const float g = decay[e / per_head];
    float* st = state + (size_t)seq_slot[b] * heads * per_head + e;
    float s = *st;
    for (int c = 0; c * chunk < n_new; ++c) {
        float* at = starts + ((size_t)b * max_chunks + c) * heads * per_head + e;
        const float local = *at;
        *at = s;
        s = fmaf(powf(g, (float)min(chunk, n_new - c * chunk)), s, local);
    }
    *st = s;
}

template <typename T>
static void retention_launch(hipStream_t stream, dim3 grid, int threads, int mode, int chunk, int max_chunks, float* starts,
                             const T* qkvg, int row_stride, int v_off, int g_off, const float* qk, const float* decay,
                             float eps, float* state, const int* seq_slot, const int* seq_new,
                             const int* cu_new, int heads, int dim, int vdim, T* out, int act, int joined, float* raw) {
#define RET_CASE(D) { if (threads <= 256) retention_kernel<T, D, 256><<<grid, threads, 0, stream>>>(mode, chunk, max_chunks, starts, qkvg, \
            row_stride, v_off, g_off, qk, decay, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, out, act, joined, raw); \
        else retention_kernel<T, D, 1024><<<grid, threads, 0, stream>>>(mode, chunk, max_chunks, starts, qkvg, \
            row_stride, v_off, g_off, qk, decay, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, out, act, joined, raw); }
    if (dim <= 32) RET_CASE(32)
    else if (dim <= 64) RET_CASE(64)
    else if (dim <= 128) RET_CASE(128)
    else RET_CASE(256)
#undef RET_CASE
}

// qk: room for n_tokens * heads * 2 * pad floats (the rotated q and k; pad = palm_retention_pad(dim)).  chunk == 0: every sequence's run in one block
// per head.  Else `starts` holds n_seqs * max_chunks * heads * dim * vdim floats, max_chunks = ceil(max_new / chunk).
PALM_API int palm_retention_pad(int dim) { return dim <= 32 ? 32 : dim <= 64 ? 64 : dim <= 128 ? 128 : 256; }

PALM_API int palm_retention(hipStream_t stream, const void* qkvg, int dtype, int row_stride, int q_off, int k_off, int v_off,
                            int g_off, const float* cos_t, const float* sin_t, int rot, const float* decay, float k_scale,
                            float eps, float* state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs,
                            int heads, int dim, int vdim, void* out, int max_new, int chunk, float* starts, int n_tokens,
                            float* qk, int act, int joined, float* raw) {
    PALM_CHECK(n_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0, "retention: seqs=%d heads=%d dim=%d vdim=%d", n_seqs, heads, dim, vdim);
    PALM_CHECK(dim <= 256, "retention: a key size of %d exceeds 256", dim);
    PALM_CHECK(vdim <= 1024, "retention: a value size of %d exceeds 1024", vdim);
    PALM_CHECK(rot >= 0 && rot <= dim && rot % 2 == 0, "retention: %d rotated dimensions of %d", rot, dim);
    PALM_CHECK(rot == 0 || (cos_t && sin_t), "retention: a rotation needs its cos and sin rows");
    PALM_CHECK(chunk >= 0 && (chunk == 0 || (starts && max_new > 0)), "retention: chunks of %d tokens need their starting states", chunk);
    PALM_CHECK(n_tokens >= 0 && (n_tokens == 0 || qk), "retention: the rotated q and k need their room");
    PALM_CHECK(n_tokens == 0 || (joined ? raw != nullptr : out != nullptr), "retention: the outputs need their room (32-bit rows if the heads are normed together later)");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    const int max_chunks = chunk > 0 ? (max_new + chunk - 1) / chunk : 1;
    PALM_CHECK(heads <= 65535 && (long long)n_seqs * max_chunks <= 65535, "retention: %d heads / %d sequences x %d chunks are more than one launch takes",
               heads, n_seqs, max_chunks);
    const int threads = (vdim + WAVE - 1) / WAVE * WAVE;
    dim3 grid(heads, n_seqs * max_chunks);
    const int pad = palm_retention_pad(dim);
    const long long rot_threads = (long long)n_tokens * heads * pad;
    PALM_DTYPE_SWITCH(dtype, T, {
        retention_rotate_kernel<T><<<(unsigned)((rot_threads + 255) / 256), 256, 0, stream>>>((const T*)qkvg, row_stride, q_off, k_off, cos_t,
                                                                                             sin_t, rot, k_scale, act, n_tokens, heads, dim, pad, qk);
        if (chunk == 0) {
            retention_launch<T>(stream, grid, threads, RET_WHOLE, 1 << 30, 1, nullptr, (const T*)qkvg, row_stride, v_off, g_off, qk, decay,
                                eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out, act, joined, raw);
        } else {
            retention_launch<T>(stream, grid, threads, RET_LOCAL, chunk, max_chunks, starts, (const T*)qkvg, row_stride, v_off, g_off, qk,
                                decay, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out, act, joined, raw);
            const int elems = heads * dim * vdim;
            retention_starts_kernel<<<dim3((elems + 255) / 256, n_seqs), 256, 0, stream>>>(starts, state, decay, seq_slot, seq_new, chunk,
                                                                                         max_chunks, heads, dim * vdim);
            retention_launch<T>(stream, grid, threads, RET_FROM_STARTS, chunk, max_chunks, starts, (const T*)qkvg, row_stride, v_off, g_off,
                                qk, decay, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out, act, joined, raw);
        }
    });
    PALM_LAUNCHED();
    return 0;
}

__device__ inline void ret_load4(const float* p, float (&o)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ inline void ret_load4(const bf16_t* p, float (&o)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = __builtin_bit_cast(float, v.x << 16); o[1] = __builtin_bit_cast(float, v.x & 0xffff0000u);
    o[2] = __builtin_bit_cast(float, v.y << 16); o[3] = __builtin_bit_cast(float, v.y & 0xffff0000u);
}
__device__ inline void ret_store4(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ inline void ret_store4(bf16_t* p, const float (&v)[4]) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    w.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(p) = w;
}

// ---- the joined heads normed together and gated -------------------------------------------------------------
// out[t] = raw[t] / sqrt(mean(raw[t]^2) + eps) * weight * f(gate[t]) over a token's whole row of `width` values (all
// heads), f = sigmoid (gate_act 1) or silu (gate_act 0).  raw is 32-bit; the gate lies in rows `gate_stride` elements
// apart.  One block per token.
template <typename T>
__global__ __launch_bounds__(1024) void joined_norm_gate_kernel(const float* __restrict__ raw, const float* __restrict__ weight, float eps,
                                                               const T* __restrict__ gate, int gate_stride, int gate_act, int width,
                                                               T* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const float* r = raw + t * width;
    float ss = 0.f;
    // four values a read where the row and the gate's rows allow
    const bool by_four = width % 4 == 0 && gate_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(gate) % 16) == 0;
    if (by_four) {
        for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {
            const float4 v = *reinterpret_cast<const float4*>(r + c);
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    } else {
        for (int c = threadIdx.x; c < width; c += blockDim.x) { const float v = r[c]; ss += v * v; }
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    auto gated = [&](float o, float w, float g) {
        const float f = gate_act == 1 ? 1.0f / (1.0f + expf(-g)) : g / (1.0f + expf(-g));
        return o * inv * w * f;
    };
    if (by_four) {
        for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {
            const float4 v = *reinterpret_cast<const float4*>(r + c), w = *reinterpret_cast<const float4*>(weight + c);
            float g[4];
            ret_load4(gate + t * gate_stride + c, g);
            const float y[4] = {gated(v.x, w.x, g[0]), gated(v.y, w.y, g[1]), gated(v.z, w.z, g[2]), gated(v.w, w.w, g[3])};
            ret_store4(out + t * width + c, y);
        }
    } else {
        for (int c = threadIdx.x; c < width; c += blockDim.x)
            out[t * width + c] = from_float<T>(gated(r[c], weight[c], to_float(gate[t * gate_stride + c])));
    }
}

PALM_API int palm_joined_norm_gate(hipStream_t stream, const float* raw, const float* weight, float eps, const void* gate, int dtype,
                                   int gate_stride, int gate_act, int n_tokens, int width, void* out) {
    PALM_CHECK(n_tokens >= 0 && width > 0 && gate_stride >= width, "joined_norm_gate: tokens=%d width=%d gate rows %d apart", n_tokens, width, gate_stride);
    PALM_CHECK(gate_act == 0 || gate_act == 1, "joined_norm_gate: gate activation %d is neither silu (0) nor sigmoid (1)", gate_act);
    if (n_tokens == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T,
        joined_norm_gate_kernel<T><<<n_tokens, n_tokens >= 256 ? 256 : width >= 2048 ? 1024 : width >= 1024 ? 512 : 256, 0, stream>>>(raw, weight, eps, (const T*)gate, gate_stride, gate_act, width, (T*)out));
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
