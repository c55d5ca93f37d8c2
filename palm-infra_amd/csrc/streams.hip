// A residual stream in several copies ("streams") with learned weights between them, and norms that need no statistics.
//
// The stream of a token is xs[s], s = 0 .. S-1, each `width` wide, 32-bit, laid out [tokens, S, width].  A sublayer reads
//
//   u = sum_s in[s] xs[s]                       (in absent: every weight is one, the plain sum of the streams)
//
// through a norm, and its output y goes back into all streams at once, each new stream made from all the old ones:
//
//   xs'[t] = sum_s mix[s][t] xs[s] + out[t] y        (mix is indexed [from, to])
//
// One kernel does the write of one sublayer and the read of the next: a token's row in blocks of columns, every thread four
// neighbouring columns, all S old values of a column in registers, the new ones stored (unless only some rows are read: then the stream stays as it is
// and the rows are computed for their reader alone), the weighted sum normed and rounded once.  Norms:
//
//   none   y = u
//   dyt    y = tanh(alpha u) w + b              (no mean, no variance: nothing crosses the columns)
//   rms    y = u / sqrt(mean(u^2) + eps) * w    (the sums wait in LDS for the row's factor)
//
// Everything is 32-bit but the sublayer's output as it comes in and the normed rows as they go out.
#include "common.h"

constexpr int ST_MAX = 16;                 // streams
enum StreamNorm : int { SN_NONE = 0, SN_DYT = 1, SN_RMS = 2 };

// xs[t][s][:] = x[t][:] for every s.
__global__ void streams_spread_kernel(const float* __restrict__ x, int S, int width, float* __restrict__ xs) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float v = x[t * width + c];
        for (int s = 0; s < S; ++s) xs[(t * S + s) * width + c] = v;
    }
}

PALM_API int palm_streams_spread(hipStream_t stream, const float* x, int n_tokens, int S, int width, float* xs) {
    PALM_CHECK(n_tokens >= 0 && S >= 1 && S <= ST_MAX && width > 0, "streams_spread: tokens=%d streams=%d width=%d", n_tokens, S, width);
    if (n_tokens == 0) return 0;
    streams_spread_kernel<<<n_tokens, 256, 0, stream>>>(x, S, width, xs);
    PALM_LAUNCHED();
    return 0;
}

// VEC neighbouring values of a row at a time (four where the width allows: 16-byte reads and writes of the streams).
template <int VEC> struct Pack { float v[VEC]; };
template <int VEC> __device__ inline Pack<VEC> st_load(const float* p) {
    Pack<VEC> r;
    if constexpr (VEC == 4) { const float4 t = *reinterpret_cast<const float4*>(p); r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w; }
    else r.v[0] = p[0];
    return r;
}
template <int VEC> __device__ inline Pack<VEC> st_load(const bf16_t* p) {
    Pack<VEC> r;
    if constexpr (VEC == 4) {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        r.v[0] = __builtin_bit_cast(float, t.x << 16); r.v[1] = __builtin_bit_cast(float, t.x & 0xffff0000u);
        r.v[2] = __builtin_bit_cast(float, t.y << 16); r.v[3] = __builtin_bit_cast(float, t.y & 0xffff0000u);
    } else r.v[0] = to_float(p[0]);
    return r;
}
template <int VEC> __device__ inline void st_store(float* p, const Pack<VEC>& r) {
    if constexpr (VEC == 4) *reinterpret_cast<float4*>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
    else p[0] = r.v[0];
}
template <int VEC> __device__ inline void st_store(bf16_t* p, const Pack<VEC>& r) {
    if constexpr (VEC == 4) {
        uint2 w;
        w.x = (uint32_t)f32_to_bf16(r.v[0]).bits | ((uint32_t)f32_to_bf16(r.v[1]).bits << 16);
        w.y = (uint32_t)f32_to_bf16(r.v[2]).bits | ((uint32_t)f32_to_bf16(r.v[3]).bits << 16);
        *reinterpret_cast<uint2*>(p) = w;
    } else p[0] = f32_to_bf16(r.v[0]);
}

// grid (rows, blocks of columns): a norm that needs the whole row (rms) has one block a row, which walks over the columns;
// the others cut a row into blocks of columns, so that a step of few rows still fills the chip.
template <typename TY, typename TO, int VEC, int SMAX>
__global__ __launch_bounds__(1024) void streams_mix_norm_kernel(
    float* __restrict__ xs, int S, int width, const TY* __restrict__ y, const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, int norm_kind, const float* __restrict__ nw, const float* __restrict__ nb, float alpha, float eps,
    const int* __restrict__ rows, int update, TO* __restrict__ out) {
    extern __shared__ float u_s[];                           // [width] for the rms norm, else nothing
    __shared__ float mix_s[SMAX * SMAX], out_s[SMAX], in_s[SMAX];
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    const size_t t = rows ? (size_t)rows[r] : r;
    for (int i = threadIdx.x; i < S * S; i += blockDim.x) mix_s[i] = y ? mix[i] : 0.f;
    for (int i = threadIdx.x; i < S; i += blockDim.x) { out_s[i] = y ? out_w[i] : 0.f; in_s[i] = in_w ? in_w[i] : 1.f; }
    __syncthreads();
    float* base = xs + t * S * width;
    float ss = 0.f;
    for (int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC; c < width; c += gridDim.y * blockDim.x * VEC) {
        Pack<VEC> old[SMAX];
#pragma unroll
        for (int s = 0; s < SMAX; ++s)
            if (s < S) old[s] = st_load<VEC>(base + (size_t)s * width + c);
        Pack<VEC> u;
#pragma unroll
        for (int e = 0; e < VEC; ++e) u.v[e] = 0.f;
        if (y) {
            const Pack<VEC> yv = st_load<VEC>(y + t * width + c);
#pragma unroll
            for (int to = 0; to < SMAX; ++to) {
                if (to < S) {
                    Pack<VEC> v;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) v.v[e] = out_s[to] * yv.v[e];
#pragma unroll
                    for (int from = 0; from < SMAX; ++from)
                        if (from < S) {
#pragma unroll
                            for (int e = 0; e < VEC; ++e) v.v[e] = fmaf(mix_s[from * S + to], old[from].v[e], v.v[e]);
                        }
                    if (update) st_store<VEC>(base + (size_t)to * width + c, v);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) u.v[e] = fmaf(in_s[to], v.v[e], u.v[e]);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
                if (s < S) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) u.v[e] = fmaf(in_s[s], old[s].v[e], u.v[e]);
                }
        }
        if (!out) continue;
        if (norm_kind == SN_RMS) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { u_s[c + e] = u.v[e]; ss = fmaf(u.v[e], u.v[e], ss); }
        } else {
            if (norm_kind == SN_DYT) {
                const Pack<VEC> w = st_load<VEC>(nw + c);
#pragma unroll
                for (int e = 0; e < VEC; ++e) u.v[e] = fmaf(tanhf(alpha * u.v[e]), w.v[e], nb ? nb[c + e] : 0.f);
            }
            st_store<VEC>(out + r * width + c, u);
        }
    }
    if (out && norm_kind == SN_RMS) {
        const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);       // (its barrier also orders u_s)
        for (int c = threadIdx.x; c < width; c += blockDim.x) out[r * width + c] = from_float<TO>(u_s[c] * inv * nw[c]);
    }
}

// xs float32 [n_tokens, S, width], updated in place if `update`.  y: null (nothing is written: a read alone), or the sublayer's
// output [n_tokens, width] with mix float32 [S, S] ([from, to]) and out_w float32 [S].  in_w: float32 [S] or null (ones).
// rows: null (every token, n_rows = n_tokens) or the n_rows tokens to read.  out: null (a write alone), or [n_rows, width].
PALM_API int palm_streams_mix_norm(hipStream_t stream, float* xs, int n_tokens, int S, int width, const void* y, int y_dtype,
                                   const float* mix, const float* out_w, const float* in_w, int norm_kind, const float* nw,
                                   const float* nb, float alpha, float eps, const int* rows, int n_rows, int update, void* out,
                                   int out_dtype) {
    PALM_CHECK(n_tokens >= 0 && n_rows >= 0 && S >= 1 && S <= ST_MAX && width > 0, "streams_mix_norm: tokens=%d rows=%d streams=%d width=%d",
               n_tokens, n_rows, S, width);
    PALM_CHECK(!y || (mix && out_w), "streams_mix_norm: a sublayer's output needs the weights that spread it");
    PALM_CHECK(norm_kind >= SN_NONE && norm_kind <= SN_RMS, "streams_mix_norm: norm kind %d", norm_kind);
    PALM_CHECK(!out || norm_kind == SN_NONE || nw, "streams_mix_norm: a norm needs its weight");
    PALM_CHECK(rows || n_rows == n_tokens, "streams_mix_norm: without a selection every token is a row (%d of %d)", n_rows, n_tokens);
    PALM_CHECK(!(update && rows), "streams_mix_norm: a selection of rows leaves the stream as it is");
    PALM_CHECK(y || out, "streams_mix_norm: nothing to do");
    PALM_CHECK(norm_kind != SN_RMS || width <= 16384, "streams_mix_norm: the rms norm holds a row of at most 16384 values, not %d", width);
    if (n_rows == 0) return 0;
    const bool whole_row = out && norm_kind == SN_RMS;
    const int vec = width % 4 == 0 ? 4 : 1;
    int threads = 256, col_blocks = 1;
    if (whole_row) threads = n_rows >= 256 ? 256 : width >= 4096 * vec ? 1024 : width >= 1024 * vec ? 512 : 256;
    else col_blocks = (width + threads * vec - 1) / (threads * vec);
    PALM_CHECK(col_blocks <= 65535, "streams_mix_norm: a width of %d is more than one launch takes", width);
    const size_t lds = whole_row ? (size_t)width * sizeof(float) : 0;
    const dim3 grid(n_rows, col_blocks);
#define ST_CASE(V, SM) streams_mix_norm_kernel<TY, TO, V, SM><<<grid, threads, lds, stream>>>(xs, S, width, (const TY*)y, mix, out_w, in_w, norm_kind, \
        nw, nb, alpha, eps, rows, update, (TO*)out)
    PALM_DTYPE_SWITCH(y_dtype, TY, {
        PALM_DTYPE_SWITCH(out_dtype, TO, {
            // (few streams, the usual case: their values stay in a thread's registers with room to spare)
            if (vec == 4 && S <= 4) ST_CASE(4, 4); else if (vec == 4 && S <= 8) ST_CASE(4, 8); else if (S <= 4) ST_CASE(1, 4); else ST_CASE(1, ST_MAX);
        });
    });
#undef ST_CASE
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
