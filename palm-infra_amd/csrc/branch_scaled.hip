// Branches whose outputs are multiplied by a learned vector before they are added to the residual stream, and the
// feed-forward activation with capped operands.
//
//   x[r] += ls * (c0 * d0[r] + c1 * d1[r])          ls: float32 [width] ("layer scale"); c0, c1: fixed weights of the
//   out[r] = x[r] / sqrt(mean(x[r]^2) + eps) * w     branch's one or two terms; everything 32-bit; w: the norm that reads
//                                                    the stream next (none: the sum alone is made)
//
//   y = g * sigmoid(slope * g) * (u + shift),   g = min(gate, limit),   u = clamp(up, -limit, limit)
#include "common.h"

// Four values of a row at a time (16 bytes of float32, 8 of bfloat16) where the sizes allow.
__device__ inline void load4(const float* p, float (&o)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ inline void load4(const bf16_t* p, float (&o)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = __builtin_bit_cast(float, v.x << 16); o[1] = __builtin_bit_cast(float, v.x & 0xffff0000u);
    o[2] = __builtin_bit_cast(float, v.y << 16); o[3] = __builtin_bit_cast(float, v.y & 0xffff0000u);
}
__device__ inline void store4(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ inline void store4(bf16_t* p, const float (&v)[4]) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    w.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(p) = w;
}

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
    const bool by_four = width % 4 == 0;
    if (by_four) {
        for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {
            float a[4], b[4] = {0.f, 0.f, 0.f, 0.f}, l[4] = {1.f, 1.f, 1.f, 1.f}, xv[4], v[4];
            load4(d0 + r * width + c, a);
            if (d1) load4(d1 + r * width + c, b);
            if (ls) load4(ls + c, l);
            load4(xr + c, xv);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float d = c0 * a[i];
                if (d1) d = fmaf(c1, b[i], d);
                v[i] = fmaf(l[i], d, xv[i]);
                ss += v[i] * v[i];
            }
            if (update) store4(xr + c, v);
            store4(sums + c, v);
        }
    } else {
        for (int c = threadIdx.x; c < width; c += blockDim.x) {
            float d = c0 * to_float(d0[r * width + c]);
            if (d1) d = fmaf(c1, to_float(d1[r * width + c]), d);
            const float v = fmaf(ls ? ls[c] : 1.f, d, xr[c]);
            if (update) xr[c] = v;
            sums[c] = v;
            ss += v * v;
        }
    }
    if (!w) return;
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    TO* o = out + (size_t)blockIdx.x * width;
    if (by_four) {
        for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {     // (a thread reads back what it wrote itself)
            float v[4], wv[4];
            load4(sums + c, v);
            load4(w + c, wv);
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = v[i] * inv * wv[i];
            store4(o + c, v);
        }
    } else {
        for (int c = threadIdx.x; c < width; c += blockDim.x) o[c] = from_float<TO>(sums[c] * inv * w[c]);
    }
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
    const int threads = n_out >= 256 ? 256 : width >= 4096 ? 1024 : width >= 2048 ? 512 : 256;
    PALM_DTYPE_SWITCH(d_dtype, TD, {
        PALM_DTYPE_SWITCH(out_dtype, TO,
            add_scaled_normed_kernel<TD, TO><<<n_out, threads, lds, stream>>>(x, (const TD*)d0, c0, (const TD*)d1, c1, ls, w, eps, rows, width,
                                                                         update, (TO*)out));
    });
    PALM_LAUNCHED();
    return 0;
}

// gate_up [n, 2 ff]: a row's gate values, then its up values.
__device__ inline float capped(float gate, float up, float limit, float slope, float shift) {
    const float g = fminf(gate, limit);
    const float u = fminf(fmaxf(up, -limit), limit);
    return g * (1.0f / (1.0f + expf(-slope * g))) * (u + shift);
}

// A row a blockIdx.y; a thread takes four columns at a time if the inner size is a multiple of four, else one.
template <typename T>
__global__ void capped_gate_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int ff, float limit, float slope, float shift) {
    const size_t r = blockIdx.y;
    const T* row = gate_up + r * 2 * ff;
    if (ff % 4 == 0) {
        const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
        if (c >= ff) return;
        float g[4], u[4], y[4];
        load4(row + c, g);
        load4(row + ff + c, u);
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = capped(g[i], u[i], limit, slope, shift);
        store4(out + r * ff + c, y);
    } else {
        for (int c = blockIdx.x * blockDim.x * 4 + threadIdx.x; c < min(ff, (int)(blockIdx.x + 1) * (int)blockDim.x * 4); c += blockDim.x)
            out[r * ff + c] = from_float<T>(capped(to_float(row[c]), to_float(row[ff + c]), limit, slope, shift));
    }
}

PALM_API int palm_capped_gate(hipStream_t stream, const void* gate_up, void* out, int dtype, int n, int ff, float limit, float slope,
                              float shift) {
    PALM_CHECK(n >= 0 && ff > 0 && limit > 0.f, "capped_gate: rows=%d ff=%d limit=%g", n, ff, (double)limit);
    if (n == 0) return 0;
    PALM_CHECK(n <= 65535, "capped_gate: %d rows are more than one launch takes", n);
    const dim3 grid((ff + 1023) / 1024, n);                      // a block of 256 threads takes 1,024 columns of a row
    PALM_DTYPE_SWITCH(dtype, T,
        capped_gate_kernel<T><<<grid, 256, 0, stream>>>((const T*)gate_up, (T*)out, ff, limit, slope, shift));
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
