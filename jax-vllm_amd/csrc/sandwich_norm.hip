// Norms of a layer arrangement that norms a sublayer's output before it joins the residual
// stream ("sandwich": x += N_b(f(N_a(x)))), and the gated norm behind a recurrent mixer.
// All sums, inverse roots and the residual stream are float.
#include "common.h"

// ---------------------------------------------------------------- post-norm + residual add + next pre-norm
// Row r = rows ? rows[i] : i.
//   v   = (y ? y[r] : 0) + parts[0][r] + parts[1][r] + ...       (the sublayer's output; parts added in order)
//   x   = h[r] + v * rsqrt(mean(v^2) + eps) * wb                 (float)
//   if (!rows) h[r] = x
//   if (out)   out[i] = T( x * rsqrt(mean(x^2) + eps_out) * w )
// One block per output row; the row is kept in LDS between the passes (hidden floats).
template <typename T>
__global__ void __launch_bounds__(256)
postnorm_add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ y, const float* __restrict__ parts,
                            int n_parts, long long part_stride, const float* __restrict__ wb,
                            const float* __restrict__ w, T* __restrict__ out, const int* __restrict__ rows,
                            int hidden, float eps, float eps_out) {
  extern __shared__ float row[];
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float* hr = h + r * hidden;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = y ? to_f32(y[r * hidden + c]) : 0.f;
    for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + r * hidden + c];
    row[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv_b = rsqrtf(ss / (float)hidden + eps);
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float x = hr[c] + row[c] * inv_b * wb[c];
    if (!rows) hr[c] = x;
    row[c] = x;
    ss2 += x * x;
  }
  if (!out) return;
  ss2 = block_sum(ss2, red);
  const float inv = rsqrtf(ss2 / (float)hidden + eps_out);
  T* o = out + i * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) o[c] = from_f32<T>(row[c] * inv * w[c]);
}

// ---------------------------------------------------------------- norm of float rows times a sigmoid gate
//   out[t, c] = T( o[t, c] * rsqrt(mean_c(o[t]^2) + eps) * w[c] * sigmoid(g[t * g_stride + c]) )
// o is float (the output of a recurrence), g lives in a wider row of the activation type.
template <typename T>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g,
                     long long g_stride, const float* __restrict__ w, int width, float eps) {
  __shared__ float red[32];
  const long long t = blockIdx.x;
  const float* x = o + t * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) ss += x[c] * x[c];
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float gate = 1.f / (1.f + expf(-to_f32(g[t * g_stride + c])));
    out[t * width + c] = from_f32<T>(x[c] * inv * w[c] * gate);
  }
}

#define DEFINE_SANDWICH(SUF, T)                                                                          \
  extern "C" int jv_postnorm_add_rmsnorm_##SUF(float* h, const void* y, const float* parts, int n_parts, \
                                               long long part_stride, const float* wb, const float* w,   \
                                               void* out, const int* rows, int n_out, int hidden,        \
                                               float eps, float eps_out, void* stream) {                 \
    if (n_out <= 0 || hidden <= 0) return 0;                                                             \
    if ((!y && n_parts <= 0) || hidden > 16384) return (int)hipErrorInvalidValue;                        \
    hipLaunchKernelGGL(postnorm_add_rmsnorm_kernel<T>, dim3(n_out), dim3(256), hidden * sizeof(float),   \
                       (hipStream_t)stream, h, (const T*)y, parts, n_parts, part_stride, wb, w, (T*)out, \
                       rows, hidden, eps, eps_out);                                                      \
    return JV_LAUNCH_CHECK();                                                                            \
  }                                                                                                      \
  extern "C" int jv_gated_rmsnorm_##SUF(void* out, const float* o, const void* g, long long g_stride,    \
                                        const float* w, int n, int width, float eps, void* stream) {     \
    if (n <= 0 || width <= 0) return 0;                                                                  \
    hipLaunchKernelGGL(gated_rmsnorm_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t)stream, (T*)out, o,  \
                       (const T*)g, g_stride, w, width, eps);                                            \
    return JV_LAUNCH_CHECK();                                                                            \
  }

DEFINE_SANDWICH(bf16, bf16_t)
DEFINE_SANDWICH(f32, float)
