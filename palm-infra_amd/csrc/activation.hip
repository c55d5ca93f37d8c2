// Elementwise activations of plain feed-forwards (down(act(up(h)))), 32-bit inside:
//
//   relu_squared   max(z, 0)^2
//   gelu_erf       z/2 (1 + erf(z / sqrt 2))
//   gelu_tanh      z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
#include "common.h"

enum Activation : int { ACT_RELU_SQUARED = 0, ACT_GELU_ERF = 1, ACT_GELU_TANH = 2 };

template <typename T>
__global__ void activation_kernel(const T* __restrict__ z, T* __restrict__ out, int kind, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = to_float(z[i]);
    float r;
    if (kind == ACT_RELU_SQUARED) { const float p = fmaxf(v, 0.f); r = p * p; }
    else if (kind == ACT_GELU_ERF) r = 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
    else r = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    out[i] = from_float<T>(r);
}

PALM_API int palm_activation(hipStream_t stream, const void* z, void* out, int dtype, int kind, long long n) {
    PALM_CHECK(n >= 0 && kind >= ACT_RELU_SQUARED && kind <= ACT_GELU_TANH, "activation: n=%lld kind=%d", n, kind);
    if (n == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T, activation_kernel<T><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((const T*)z, (T*)out, kind, n));
    PALM_LAUNCHED();
    return 0;
}

PALM_DEFINE_LAST_ERROR()
