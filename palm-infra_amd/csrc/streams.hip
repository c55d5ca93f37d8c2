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
// One kernel does the write of one sublayer and the read of the next: a block a token, every thread a few columns, all S
// old values of a column in registers, the new ones stored (unless only some rows are read: then the stream stays as it is
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

template <typename TY, typename TO>
__global__ __launch_bounds__(1024) void streams_mix_norm_kernel(
    float* __restrict__ xs, int S, int width, const TY* __restrict__ y, const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, int norm_kind, const float* __restrict__ nw, const float* __restrict__ nb, float alpha, float eps,
    const int* __restrict__ rows, int update, TO* __restrict__ out) {
    extern __shared__ float u_s[];                           // [width] for the rms norm, else nothing
    __shared__ float mix_s[ST_MAX * ST_MAX], out_s[ST_MAX], in_s[ST_MAX];
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    const size_t t = rows ? (size_t)rows[r] : r;
    for (int i = threadIdx.x; i < S * S; i += blockDim.x) mix_s[i] = y ? mix[i] : 0.f;
    for (int i = threadIdx.x; i < S; i += blockDim.x) { out_s[i] = y ? out_w[i] : 0.f; in_s[i] = in_w ? in_w[i] : 1.f; }
    __syncthreads();
    float* base = xs + t * S * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float old[ST_MAX];
#pragma unroll
        for (int s = 0; s < ST_MAX; ++s) old[s] = s < S ? base[(size_t)s * width + c] : 0.f;
        float u = 0.f;
        if (y) {
            const float yv = to_float(y[t * width + c]);
#pragma unroll
            for (int to = 0; to < ST_MAX; ++to) {
                if (to < S) {
                    float v = out_s[to] * yv;
#pragma unroll
                    for (int from = 0; from < ST_MAX; ++from)
                        if (from < S) v = fmaf(mix_s[from * S + to], old[from], v);
                    if (update) base[(size_t)to * width + c] = v;
                    u = fmaf(in_s[to], v, u);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < ST_MAX; ++s)
                if (s < S) u = fmaf(in_s[s], old[s], u);
        }
        if (!out) continue;
        if (norm_kind == SN_RMS) {
            u_s[c] = u;
            ss = fmaf(u, u, ss);
        } else {
            const float v = norm_kind == SN_DYT ? fmaf(tanhf(alpha * u), nw[c], nb ? nb[c] : 0.f) : u;
            out[r * width + c] = from_float<TO>(v);
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
    const int threads = n_rows >= 256 ? 256 : width >= 4096 ? 1024 : width >= 1024 ? 512 : 256;
    const size_t lds = out && norm_kind == SN_RMS ? (size_t)width * sizeof(float) : 0;
    PALM_DTYPE_SWITCH(y_dtype, TY, {
        PALM_DTYPE_SWITCH(out_dtype, TO, {
            streams_mix_norm_kernel<TY, TO><<<n_rows, threads, lds, stream>>>(xs, S, width, (const TY*)y, mix, out_w, in_w, norm_kind, nw, nb,
                                                                             alpha, eps, rows, update, (TO*)out);
        });
    });
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
