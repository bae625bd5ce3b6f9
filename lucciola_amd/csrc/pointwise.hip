// Element-wise kernels of the parts that came after the first architecture: the Dynamic Tanh
// norm (with the residual addition folded in, as the RMSNorm kernel has it), a vector added to
// every row of the residual stream, and the activations of the two-matrix feed-forwards.
// All arithmetic is float32; only loads and stores have the tensors' types.
//   dynamic tanh   y = tanh(alpha v) w + b,  v = h (+ delta)
//   gelu (tanh)    0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
//   relu squared   max(z, 0)^2
#include "common.h"

#include "activations.h"

namespace lc {

// One workgroup per output row r; src row = rows ? rows[r] : r.
//   v = h[src] (+ delta[src]);  if (write_h) h[src] = v;  out[r] = tanh(alpha v) w + b
template <typename T>
__global__ void dynamic_tanh_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                    const int* __restrict__ rows, const float* __restrict__ w,
                                    const float* __restrict__ b, float alpha, T* __restrict__ out, int n,
                                    int write_h) {
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* hr = h + (size_t)src * n;
    const T* dr = delta ? delta + (size_t)src * n : nullptr;
    T* o = out + (size_t)r * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i];
        if (dr) {
            v += to_f32(dr[i]);
            if (write_h) hr[i] = v;
        }
        o[i] = from_f32<T>(fmaf(tanhf(alpha * v), w[i], b[i]));
    }
}

// h[t] += delta[t] + vec, for every row t
template <typename T>
__global__ void stream_add_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                  const float* __restrict__ vec, int n, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float v = h[idx];
        if (delta) v += to_f32(delta[idx]);
        h[idx] = v + vec[idx % n];
    }
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ x, int kind, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x)
        x[idx] = from_f32<T>(activate(to_f32(x[idx]), kind));
}

static int blocks_for(size_t total) { return (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192); }

}  // namespace lc

using namespace lc;

LC_API int lc_dynamic_tanh(float* h, const void* delta, const int* rows, const float* w, const float* b,
                           float alpha, void* out, int dt, int R, int n, int write_h, hipStream_t stream) {
    LC_CHECK(R >= 0 && n > 0, "dynamic_tanh: bad sizes R=%d n=%d", R, n);
    if (R == 0) return 0;
    LC_CHECK(h && w && b && out, "dynamic_tanh: null pointer");
    LC_CHECK(!(rows && write_h), "dynamic_tanh: gathered rows cannot be written back");
    // a row's entries are independent: with few rows, as many threads a row as it has pairs of
    // entries, so that no thread walks the row load after load
    const int threads = (R <= 256 && n >= 2048) ? 1024 : (n >= 512 ? 256 : (n >= 128 ? 128 : 64));
    if (dt == DT_F32)
        dynamic_tanh_kernel<float><<<R, threads, 0, stream>>>(h, (const float*)delta, rows, w, b, alpha, (float*)out, n, write_h);
    else if (dt == DT_BF16)
        dynamic_tanh_kernel<bf16><<<R, threads, 0, stream>>>(h, (const bf16*)delta, rows, w, b, alpha, (bf16*)out, n, write_h);
    else
        LC_CHECK(false, "dynamic_tanh: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("dynamic_tanh");
    return 0;
}

LC_API int lc_stream_add(float* h, const void* delta, int dt, const float* vec, int T, int n, hipStream_t stream) {
    LC_CHECK(T >= 0 && n > 0, "stream_add: bad sizes T=%d n=%d", T, n);
    if (T == 0) return 0;
    LC_CHECK(h && vec, "stream_add: null pointer");
    const size_t total = (size_t)T * n;
    if (dt == DT_F32)
        stream_add_kernel<float><<<blocks_for(total), 256, 0, stream>>>(h, (const float*)delta, vec, n, total);
    else if (dt == DT_BF16)
        stream_add_kernel<bf16><<<blocks_for(total), 256, 0, stream>>>(h, (const bf16*)delta, vec, n, total);
    else
        LC_CHECK(false, "stream_add: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("stream_add");
    return 0;
}

// kind: 1 gelu (tanh form), 2 relu squared; in place
LC_API int lc_activation(void* x, int dt, int kind, long long total, hipStream_t stream) {
    LC_CHECK(total >= 0 && (kind == ACT_GELU_TANH || kind == ACT_RELU_SQUARED), "activation: bad arguments");
    if (total == 0) return 0;
    LC_CHECK(x, "activation: null pointer");
    if (dt == DT_F32)
        activation_kernel<float><<<blocks_for((size_t)total), 256, 0, stream>>>((float*)x, kind, (size_t)total);
    else if (dt == DT_BF16)
        activation_kernel<bf16><<<blocks_for((size_t)total), 256, 0, stream>>>((bf16*)x, kind, (size_t)total);
    else
        LC_CHECK(false, "activation: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("activation");
    return 0;
}
