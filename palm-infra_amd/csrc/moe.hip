// A feed-forward of routed experts: every token goes through `top` of `experts` small gated feed-forwards.
//
//   route      from a token's router logits (32-bit): the `top` largest (the lower index wins a tie), and as their
//              weights the softmax over those logits alone
//   few rows (a decode step): nothing is planned on the host, every (token, choice) reads its expert's weights itself
//     expert_gate_up   mid[t, c, f] = silu(G_e h_t)[f] * (U_e h_t)[f],  e = chosen[t, c]           (32-bit)
//     expert_down      out[t, :] = sum_c weight[t, c] * D_e mid[t, c, :]  in the order of c        (32-bit)
//   An expert's form: gated (silu(G h) * (U h), the gate rows before the up rows) or plain with the exact gelu (gelu(U h)).
//
//   route, scored: the scores are sigmoid(logit); the choice is made by score plus a correction per expert; experts lie in
//              equal groups of neighbours, a group's rank is the sum of its two largest corrected scores, and only experts
//              of the best `keep` groups can be chosen; the weights are the chosen experts' scores (without the correction)
//              over their sum, times a scale
//   many rows (a prompt): the host groups the (token, choice) pairs by expert, the products are the library's
//     gather_rows      xs[p, :] = h[src[p], :]
//     scatter_add      out[rows[i], :] += weight[i] * y[i, :]      (an expert's rows are distinct tokens: no two
//                      threads meet, and the experts are added one after the other)
#include "common.h"

constexpr int ROUTE_MAX_PER_LANE = 8;            // up to 512 experts

// Eight neighbouring values of a row as floats: one 16-byte read of bfloat16, two of float32.
__device__ inline void load8(const bf16_t* p, float (&v)[8]) {
    const uint4 t = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xffff0000u);
    v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xffff0000u);
}
__device__ inline void load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// One wave per token.
__global__ __launch_bounds__(WAVE) void moe_route_kernel(const float* __restrict__ logits, int experts, int top,
                                                         int* __restrict__ chosen, float* __restrict__ weight) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x;
    float z[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
        const int e = i * WAVE + lane;
        z[i] = e < experts ? logits[t * experts + e] : -INFINITY;
    }
    float first = 0.f, sum = 0.f, mine = 0.f;
    for (int c = 0; c < top; ++c) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
            const int e = i * WAVE + lane;
            if (e < experts && (z[i] > best || (z[i] == best && e < at))) { best = z[i]; at = e; }
        }
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, WAVE);
            const int oa = __shfl_xor(at, off, WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (c == 0) first = best;
        const float p = expf(best - first);                  // the first is the largest
        sum += p;
        if (lane == c) mine = p;                             // lane c keeps choice c's weight
        if (lane == 0) chosen[t * top + c] = at;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i)
            if (i * WAVE + lane == at) z[i] = -INFINITY;
    }
    if (lane < top) weight[t * top + lane] = mine / sum;
}

// One wave per token.  logits: rows `stride` apart (other columns may follow the experts').
__device__ inline float moe_gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

__global__ __launch_bounds__(WAVE) void moe_route_scored_kernel(const float* __restrict__ logits, int stride, int experts, int top,
                                                                const float* __restrict__ correction, int groups, int keep, float scale,
                                                                int* __restrict__ chosen, float* __restrict__ weight) {
    __shared__ float choice_s[ROUTE_MAX_PER_LANE * WAVE];
    __shared__ float group_s[ROUTE_MAX_PER_LANE * WAVE];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x;
    float s[ROUTE_MAX_PER_LANE], z[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
        const int e = i * WAVE + lane;
        s[i] = e < experts ? 1.0f / (1.0f + expf(-logits[t * stride + e])) : 0.f;
        z[i] = e < experts ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;
        if (e < experts) choice_s[e] = z[i];
    }
    if (groups > 1) {
        const int size = experts / groups;
        __syncthreads();
        for (int g = lane; g < groups; g += WAVE) {                    // the sum of the group's two largest
            float a = -INFINITY, b = -INFINITY;
            for (int j = 0; j < size; ++j) {
                const float v = choice_s[g * size + j];
                if (v > a) { b = a; a = v; } else if (v > b) b = v;
            }
            group_s[g] = size > 1 ? a + b : a;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
            const int e = i * WAVE + lane;
            if (e >= experts) continue;
            const int g = e / size;
            const float mine = group_s[g];
            int better = 0;                                            // groups ahead of this one (the lower index wins a tie)
            for (int o = 0; o < groups; ++o) better += group_s[o] > mine || (group_s[o] == mine && o < g);
            if (better >= keep) z[i] = -INFINITY;
        }
    }
    float sum = 0.f, mine = 0.f;
    for (int c = 0; c < top; ++c) {
        float best = -INFINITY, score = 0.f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
            const int e = i * WAVE + lane;
            if (e < experts && (z[i] > best || (z[i] == best && e < at))) { best = z[i]; at = e; score = s[i]; }
        }
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, WAVE), os = __shfl_xor(score, off, WAVE);
            const int oa = __shfl_xor(at, off, WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; score = os; }
        }
        sum += score;
        if (lane == c) mine = score;
        if (lane == 0) chosen[t * top + c] = at;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i)
            if (i * WAVE + lane == at) z[i] = -INFINITY;
    }
    if (lane < top) weight[t * top + lane] = mine / (sum + 1e-20f) * scale;
}

// grid (blocks of rows of the expert's inner size, top, tokens); a wave computes a gate row and its up row at a time.
constexpr int MOE_THREADS = 256;

template <typename T, typename TW>
__global__ __launch_bounds__(MOE_THREADS) void expert_gate_up_kernel(const T* __restrict__ h, const TW* __restrict__ gate_up,
                                                                     const int* __restrict__ chosen, int top, int width, int ff,
                                                                     int rows_per_block, int form, float* __restrict__ mid) {
    extern __shared__ float h_s[];                  // [width]
    const int t = blockIdx.z, c = blockIdx.y;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = MOE_THREADS / WAVE;
    for (int d = threadIdx.x; d < width; d += MOE_THREADS) h_s[d] = to_float(h[(size_t)t * width + d]);
    __syncthreads();
    const int e = chosen[(size_t)t * top + c];
    const bool gated = form == 0;                   // else: up rows alone, through the exact gelu
    const TW* w = gate_up + (size_t)e * (gated ? 2 : 1) * ff * width;
    const int f_end = min(ff, (int)(blockIdx.x + 1) * rows_per_block);
    // Two rows of the first matrix are under way at a time in both forms: an inner value's gate row and up row, or (plain)
    // the up rows of two inner values, the wave's own and the one n_waves further on.
    const int step = gated ? n_waves : 2 * n_waves;
    for (int f = blockIdx.x * rows_per_block + wave; f < f_end; f += step) {
        const int f2 = f + n_waves;                                     // (plain form) the second inner value; beyond the block's rows: not kept
        const TW* ur = gated ? w + (size_t)(ff + f) * width : w + (size_t)f * width;
        const TW* gr = gated ? w + (size_t)f * width : w + (size_t)min(f2, ff - 1) * width;
        float g = 0.f, u = 0.f;
        if (width % 8 == 0) {                       // rows start on 16 bytes: eight values a lane and read
            for (int d = lane * 8; d < width; d += WAVE * 8) {
                float gv[8], uv[8];
                load8(ur + d, uv);
                load8(gr + d, gv);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float hv = h_s[d + i];
                    g = fmaf(gv[i], hv, g);
                    u = fmaf(uv[i], hv, u);
                }
            }
        } else {
            for (int d = lane; d < width; d += WAVE) {
                const float hv = h_s[d];
                g = fmaf(to_float(gr[d]), hv, g);
                u = fmaf(to_float(ur[d]), hv, u);
            }
        }
        u = wave_sum(u);
        g = wave_sum(g);
        if (lane == 0) {
            float* m = mid + ((size_t)t * top + c) * ff;
            if (gated) {
                m[f] = g / (1.0f + expf(-g)) * u;
            } else {
                m[f] = moe_gelu_erf(u);
                if (f2 < f_end) m[f2] = moe_gelu_erf(g);
            }
        }
    }
}

// grid (blocks of output rows, tokens); a wave computes one output value at a time, the choices one after the other.
template <typename TW>
__global__ __launch_bounds__(MOE_THREADS) void expert_down_kernel(const float* __restrict__ mid, const TW* __restrict__ down,
                                                                  const int* __restrict__ chosen, const float* __restrict__ weight,
                                                                  int top, int width, int ff, int rows_per_block,
                                                                  float* __restrict__ out) {
    extern __shared__ float m_s[];                  // [top][ff]
    const int t = blockIdx.y;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = MOE_THREADS / WAVE;
    for (int i = threadIdx.x; i < top * ff; i += MOE_THREADS) m_s[i] = mid[(size_t)t * top * ff + i];
    __syncthreads();
    const int r_end = min(width, (int)(blockIdx.x + 1) * rows_per_block);
    for (int r = blockIdx.x * rows_per_block + wave; r < r_end; r += n_waves) {
        float total = 0.f;
        for (int c = 0; c < top; ++c) {
            const TW* wr = down + ((size_t)chosen[(size_t)t * top + c] * width + r) * ff;
            float acc = 0.f;
            if (ff % 8 == 0) {
                for (int f = lane * 8; f < ff; f += WAVE * 8) {
                    float wv[8];
                    load8(wr + f, wv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc = fmaf(wv[i], m_s[c * ff + f + i], acc);
                }
            } else {
                for (int f = lane; f < ff; f += WAVE) acc = fmaf(to_float(wr[f]), m_s[c * ff + f], acc);
            }
            total = fmaf(weight[(size_t)t * top + c], wave_sum(acc), total);
        }
        if (lane == 0) out[(size_t)t * width + r] = total;
    }
}

template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ h, const int* __restrict__ src, int width, T* __restrict__ xs) {
    const size_t p = blockIdx.x;
    const T* from = h + (size_t)src[p] * width;
    for (int d = threadIdx.x; d < width; d += blockDim.x) xs[p * width + d] = from[d];
}

template <typename T>
__global__ void scatter_add_kernel(const T* __restrict__ y, const int* __restrict__ rows, const float* __restrict__ weight,
                                   int width, float* __restrict__ out) {
    const size_t i = blockIdx.x;
    float* to = out + (size_t)rows[i] * width;
    const float w = weight[i];
    for (int d = threadIdx.x; d < width; d += blockDim.x) to[d] = fmaf(w, to_float(y[i * width + d]), to[d]);
}

PALM_API int palm_moe_route(hipStream_t stream, const float* logits, int n_tokens, int experts, int top, int* chosen, float* weight) {
    PALM_CHECK(n_tokens >= 0 && experts > 0 && top > 0 && top <= experts, "moe_route: n=%d experts=%d top=%d", n_tokens, experts, top);
    PALM_CHECK(experts <= ROUTE_MAX_PER_LANE * WAVE, "moe_route: %d experts exceed %d", experts, ROUTE_MAX_PER_LANE * WAVE);
    PALM_CHECK(top <= WAVE, "moe_route: %d choices a token exceed %d", top, WAVE);
    if (n_tokens == 0) return 0;
    moe_route_kernel<<<n_tokens, WAVE, 0, stream>>>(logits, experts, top, chosen, weight);
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_moe_route_scored(hipStream_t stream, const float* logits, int stride, int n_tokens, int experts, int top,
                                   const float* correction, int groups, int keep, float scale, int* chosen, float* weight) {
    PALM_CHECK(n_tokens >= 0 && experts > 0 && top > 0 && top <= experts && stride >= experts, "moe_route_scored: n=%d experts=%d top=%d stride=%d",
               n_tokens, experts, top, stride);
    PALM_CHECK(experts <= ROUTE_MAX_PER_LANE * WAVE, "moe_route_scored: %d experts exceed %d", experts, ROUTE_MAX_PER_LANE * WAVE);
    PALM_CHECK(top <= WAVE, "moe_route_scored: %d choices a token exceed %d", top, WAVE);
    PALM_CHECK(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups, "moe_route_scored: %d experts in %d groups of which %d are kept",
               experts, groups, keep);
    PALM_CHECK((long long)keep * (experts / groups) >= top, "moe_route_scored: %d groups of %d experts cannot give %d choices", keep,
               experts / groups, top);
    if (n_tokens == 0) return 0;
    moe_route_scored_kernel<<<n_tokens, WAVE, 0, stream>>>(logits, stride, experts, top, correction, groups, keep, scale, chosen, weight);
    PALM_LAUNCHED();
    return 0;
}

// out[t, :] += sigmoid(gate[t * gate_stride]) * y[t, :]: an expert that every token goes through, behind a gate of one number a token.
template <typename T>
__global__ void add_gated_rows_kernel(float* __restrict__ out, const T* __restrict__ y, const float* __restrict__ gate, int gate_stride, int width) {
    const size_t t = blockIdx.x;
    const float g = 1.0f / (1.0f + expf(-gate[t * gate_stride]));
    for (int d = threadIdx.x; d < width; d += blockDim.x) out[t * width + d] = fmaf(g, to_float(y[t * width + d]), out[t * width + d]);
}

PALM_API int palm_add_gated_rows(hipStream_t stream, float* out, const void* y, int dtype, const float* gate, int gate_stride, int n_tokens,
                                 int width) {
    PALM_CHECK(n_tokens >= 0 && width > 0 && gate_stride > 0, "add_gated_rows: n=%d width=%d gate rows %d apart", n_tokens, width, gate_stride);
    if (n_tokens == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T, add_gated_rows_kernel<T><<<n_tokens, 256, 0, stream>>>(out, (const T*)y, gate, gate_stride, width));
    PALM_LAUNCHED();
    return 0;
}

// h [n, width]; gate_up [experts, 2 ff, width] (an expert's gate rows, then its up rows; form 1: [experts, ff, width], up rows
// alone); down [experts, width, ff];
// chosen, weight [n, top]; mid: room for n * top * ff floats; out float32 [n, width].
PALM_API int palm_moe_experts(hipStream_t stream, const void* h, int dtype, const void* gate_up, const void* down, int w_dtype,
                              const int* chosen, const float* weight, int n_tokens, int top, int width, int ff, float* mid,
                              float* out, int form) {
    PALM_CHECK(form == 0 || form == 1, "moe_experts: form %d is neither gated silu (0) nor plain gelu (1)", form);
    PALM_CHECK(n_tokens >= 0 && top > 0 && width > 0 && ff > 0, "moe_experts: n=%d top=%d width=%d ff=%d", n_tokens, top, width, ff);
    PALM_CHECK(width <= 16384 && (long long)top * ff <= 16384, "moe_experts: width %d / top x ff %d x %d exceed what a block holds", width, top, ff);
    PALM_CHECK(n_tokens <= 65535 && top <= 65535, "moe_experts: %d tokens x %d choices are more than one launch takes", n_tokens, top);
    if (n_tokens == 0) return 0;
    // blocks enough to fill the chip, but no fewer than four rows a wave
    const int up_rows = max(16, (ff + 15) / 16), up_blocks = (ff + up_rows - 1) / up_rows;
    const int down_rows = max(16, (width + 63) / 64), down_blocks = (width + down_rows - 1) / down_rows;
    PALM_DTYPE_SWITCH(dtype, T, {
        PALM_DTYPE_SWITCH(w_dtype, TW, {
            expert_gate_up_kernel<T, TW><<<dim3(up_blocks, top, n_tokens), MOE_THREADS, width * sizeof(float), stream>>>(
                (const T*)h, (const TW*)gate_up, chosen, top, width, ff, up_rows, form, mid);
            expert_down_kernel<TW><<<dim3(down_blocks, n_tokens), MOE_THREADS, (size_t)top * ff * sizeof(float), stream>>>(
                mid, (const TW*)down, chosen, weight, top, width, ff, down_rows, out);
        });
    });
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_gather_rows(hipStream_t stream, const void* h, int dtype, const int* src, int n_rows, int width, void* xs) {
    PALM_CHECK(n_rows >= 0 && width > 0, "gather_rows: rows=%d width=%d", n_rows, width);
    if (n_rows == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T, gather_rows_kernel<T><<<n_rows, 256, 0, stream>>>((const T*)h, src, width, (T*)xs));
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_scatter_add(hipStream_t stream, const void* y, int dtype, const int* rows, const float* weight, int n_rows,
                              int width, float* out) {
    PALM_CHECK(n_rows >= 0 && width > 0, "scatter_add: rows=%d width=%d", n_rows, width);
    if (n_rows == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T, scatter_add_kernel<T><<<n_rows, 256, 0, stream>>>((const T*)y, rows, weight, width, out));
    PALM_LAUNCHED();
    return 0;
}
