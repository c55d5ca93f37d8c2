// Branches whose outputs are multiplied by a learned vector before they are added to the residual stream, and the
// feed-forward activation with capped operands.
//
//   x[r] += ls * (c0 * d0[r] + c1 * d1[r])          ls: float32 [width] ("layer scale"); c0, c1: fixed weights of the
//   out[r] = x[r] / sqrt(mean(x[r]^2) + eps) * w     branch's one or two terms; everything 32-bit; w: the norm that reads
//                                                    the stream next (none: the sum alone is made)
//
//   y = g * sigmoid(slope * g) * (u + shift),   g = min(gate, limit),   u = clamp(up, -limit, limit)
#include "common.h"

// One block per row that is read next (`rows` selects them; without a selection every row, and x is updated).  The
// row's sums wait in LDS between the pass that makes them and the pass that norms them.
template <typename TD, typename TO>
__global__ __launch_bounds__(1024) void add_scaled_normed_kernel(float* __restrict__ x, const TD* __restrict__ d0, float c0,
                                                                const TD* __restrict__ d1, float c1, const float* __restrict__ ls,
                                                                const float* __restrict__ w, float eps, const int* __restrict__ rows,
                                                                int width, int update, TO* __restrict__ out) {
    extern __shared__ float sums[];
    __shared__ float scratch[16];
    const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
    float* xr = x + r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float d = c0 * to_float(d0[r * width + c]);
        if (d1) d = fmaf(c1, to_float(d1[r * width + c]), d);
        const float v = fmaf(ls ? ls[c] : 1.f, d, xr[c]);
        if (update) xr[c] = v;
        sums[c] = v;
        ss += v * v;
    }
    if (!w) return;
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    TO* o = out + (size_t)blockIdx.x * width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) o[c] = from_float<TO>(sums[c] * inv * w[c]);
}

PALM_API int palm_add_scaled_normed(hipStream_t stream, float* x, const void* d0, float c0, const void* d1, float c1, int d_dtype,
                                    const float* ls, const float* w, float eps, const int* rows, int n_out, int width, int update,
                                    void* out, int out_dtype) {
    PALM_CHECK(n_out >= 0 && width > 0 && width <= 16384, "add_scaled_normed: rows=%d width=%d (at most 16384)", n_out, width);
    if (n_out == 0) return 0;
    PALM_CHECK(x && d0, "add_scaled_normed: the stream and the branch output are needed");
    PALM_CHECK(!w || out, "add_scaled_normed: a norm needs room for its output");
    PALM_CHECK(!(rows && update), "add_scaled_normed: a selection of rows leaves the stream as it is");
    PALM_CHECK(rows || update, "add_scaled_normed: without a selection of rows the stream is updated");
    const size_t lds = (size_t)width * sizeof(float);
    // few rows (a decode step): a wide row has two values a thread, short chains of loads; many rows fill the chip anyway
    const int threads = n_out >= 256 ? 256 : width >= 2048 ? 1024 : width >= 1024 ? 512 : 256;
    PALM_DTYPE_SWITCH(d_dtype, TD, {
        PALM_DTYPE_SWITCH(out_dtype, TO,
            add_scaled_normed_kernel<TD, TO><<<n_out, threads, lds, stream>>>(x, (const TD*)d0, c0, (const TD*)d1, c1, ls, w, eps, rows, width,
                                                                         update, (TO*)out));
    });
    PALM_LAUNCHED();
    return 0;
}

// gate_up [n, 2 ff]: a row's gate values, then its up values.
template <typename T>
__global__ void capped_gate_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int ff, float limit, float slope, float shift,
                                   long long count) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const long long r = i / ff;
    const int c = (int)(i % ff);
    const float g = fminf(to_float(gate_up[r * 2 * ff + c]), limit);
    const float u = fminf(fmaxf(to_float(gate_up[r * 2 * ff + ff + c]), -limit), limit);
    out[i] = from_float<T>(g * (1.0f / (1.0f + expf(-slope * g))) * (u + shift));
}

PALM_API int palm_capped_gate(hipStream_t stream, const void* gate_up, void* out, int dtype, int n, int ff, float limit, float slope,
                              float shift) {
    PALM_CHECK(n >= 0 && ff > 0 && limit > 0.f, "capped_gate: rows=%d ff=%d limit=%g", n, ff, (double)limit);
    if (n == 0) return 0;
    const long long count = (long long)n * ff;
    PALM_DTYPE_SWITCH(dtype, T,
        capped_gate_kernel<T><<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((const T*)gate_up, (T*)out, ff, limit, slope, shift, count));
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
