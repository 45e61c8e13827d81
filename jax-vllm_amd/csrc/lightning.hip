// Linear attention with a per-head decay ("lightning"): per head a matrix state in float,
//     S_t = decay_h * S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t,
// with q, k, v = silu of projections (the activation is applied as they are loaded).  The state of a
// request lives in a row of `state` [slots + 1][heads][dim][vdim] between steps; a step reads it, runs
// its tokens, and writes it back.  Columns of S (one per element of v) never mix, so a block takes one
// (request, head, slice of columns): a thread keeps up to LT_ROWS rows of one column in registers.
//
// Two kernels with the same numbers in a different order of operations:
//  * token by token (decoded tokens, short portions): S is updated and read once per token;
//  * by chunks of LC tokens (prompt portions): within a chunk
//        o_i = decay^(i+1) (S^T q_i) + sum_{j<=i} decay^(i-j) (q_i . k_j) v_j
//        S  <- decay^n S + sum_j decay^(n-1-j) k_j v_j^T                      (n tokens in the chunk)
//    so the state is touched once per chunk and the chunk's tokens run side by side.  Only
//    non-negative powers of the decay occur.  Everything is float.
#include "common.h"

#define LT_ROWS 32

__device__ __forceinline__ float lt_silu(float z) { return z / (1.f + expf(-z)); }

// grid (requests, heads, column slices); block 256 = parts x cols threads, cols a power of two
template <typename T>
__global__ void __launch_bounds__(256)
lightning_steps_kernel(float* __restrict__ out, const T* __restrict__ proj, long long ld, int q_off, int k_off,
                       int v_off, float* __restrict__ state, const int* __restrict__ slot_ids,
                       const int* __restrict__ cu_seqlens, const float* __restrict__ decay, int heads, int dim,
                       int vdim, int cols) {
  extern __shared__ float lds[];          // 2 x (q[dim] | k[dim] | v[cols]) | partial sums [parts][cols]
  const int r = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * cols;
  const int parts = blockDim.x / cols;
  const int col = threadIdx.x % cols, part = threadIdx.x / cols;
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  if (t1 <= t0) return;
  const int stage = 2 * dim + cols;
  float* red = lds + 2 * stage;
  const float lam = decay[h];
  const bool live = c0 + col < vdim;
  float* S = state + (((long long)slot_ids[r] * heads + h) * dim) * vdim + c0 + col;
  float s[LT_ROWS];
#pragma unroll
  for (int i = 0; i < LT_ROWS; ++i) {
    const int d = part + i * parts;
    s[i] = (live && d < dim) ? S[(long long)d * vdim] : 0.f;
  }
  for (int t = t0; t < t1; ++t) {
    float* buf = lds + ((t - t0) & 1) * stage;
    const T* row = proj + (long long)t * ld;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
      buf[d] = lt_silu(to_f32(row[q_off + h * dim + d]));
      buf[dim + d] = lt_silu(to_f32(row[k_off + h * dim + d]));
    }
    if (threadIdx.x < cols)
      buf[2 * dim + threadIdx.x] = (c0 + threadIdx.x < vdim) ? lt_silu(to_f32(row[v_off + h * vdim + c0 + threadIdx.x])) : 0.f;
    __syncthreads();
    const float v = buf[2 * dim + col];
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < LT_ROWS; ++i) {
      const int d = part + i * parts;
      if (d < dim) {
        s[i] = fmaf(lam, s[i], buf[dim + d] * v);
        acc = fmaf(s[i], buf[d], acc);
      }
    }
    red[part * cols + col] = acc;
    __syncthreads();
    if (part == 0 && live) {
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += red[p * cols + col];
      out[(long long)t * heads * vdim + h * vdim + c0 + col] = o;
    }
    // the next token fills the other stage; `red` is rewritten only after the barrier behind that fill
  }
#pragma unroll
  for (int i = 0; i < LT_ROWS; ++i) {
    const int d = part + i * parts;
    if (live && d < dim) S[(long long)d * vdim] = s[i];
  }
}

// ---------------------------------------------------------------- by chunks
#define LC 32        // tokens of a chunk
// grid (requests, heads, column slices of LCOLS); block 256.  LDS: q[LC][dim], k[LC][dim], v[LC][LCOLS],
// a[LC][LC + 1], S[dim][LCOLS]
#define LCOLS 32
template <typename T>
__global__ void __launch_bounds__(256)
lightning_chunks_kernel(float* __restrict__ out, const T* __restrict__ proj, long long ld, int q_off, int k_off,
                        int v_off, float* __restrict__ state, const int* __restrict__ slot_ids,
                        const int* __restrict__ cu_seqlens, const float* __restrict__ decay, int heads, int dim,
                        int vdim) {
  extern __shared__ float lds[];
  const int r = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * LCOLS;
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  if (t1 <= t0) return;
  float* qs = lds;                       // [LC][dim + 1]
  float* ks = qs + LC * (dim + 1);       // [LC][dim + 1]
  float* vs = ks + LC * (dim + 1);       // [LC][LCOLS]
  float* as = vs + LC * LCOLS;           // [LC][LC + 1]
  float* Ss = as + LC * (LC + 1);        // [dim][LCOLS]
  float* pw = Ss + dim * LCOLS;          // [LC + 1] powers of the decay
  const int tid = threadIdx.x;
  const float lam = decay[h];
  const int ncols = min(LCOLS, vdim - c0);
  float* S = state + (((long long)slot_ids[r] * heads + h) * dim) * vdim + c0;
  for (int i = tid; i < dim * LCOLS; i += 256) {
    const int d = i / LCOLS, c = i % LCOLS;
    Ss[i] = c < ncols ? S[(long long)d * vdim + c] : 0.f;
  }
  if (tid <= LC) pw[tid] = powf(lam, (float)tid);
  const int dq = dim + 1;
  for (int b0 = t0; b0 < t1; b0 += LC) {
    const int n = min(LC, t1 - b0);
    __syncthreads();                     // the chunk before is done with every buffer
    for (int i = tid; i < LC * dim; i += 256) {
      const int j = i / dim, d = i - j * dim;
      float qv = 0.f, kv = 0.f;
      if (j < n) {
        const T* row = proj + (long long)(b0 + j) * ld;
        qv = lt_silu(to_f32(row[q_off + h * dim + d]));
        kv = lt_silu(to_f32(row[k_off + h * dim + d]));
      }
      qs[j * dq + d] = qv;
      ks[j * dq + d] = kv;
    }
    for (int i = tid; i < LC * LCOLS; i += 256) {
      const int j = i / LCOLS, c = i % LCOLS;
      vs[i] = (j < n && c < ncols) ? lt_silu(to_f32(proj[(long long)(b0 + j) * ld + v_off + h * vdim + c0 + c])) : 0.f;
    }
    __syncthreads();
    // a[i][j] = decay^(i-j) q_i . k_j for j <= i, 0 otherwise: 1,024 entries, 4 a thread
    for (int e = tid; e < LC * LC; e += 256) {
      const int i = e / LC, j = e % LC;
      float dot = 0.f;
      if (j <= i && i < n) {
        for (int d = 0; d < dim; ++d) dot = fmaf(qs[i * dq + d], ks[j * dq + d], dot);
        dot *= pw[i - j];
      }
      as[i * (LC + 1) + j] = dot;
    }
    __syncthreads();
    // o[i][c] = decay^(i+1) sum_d q_i[d] S[d][c] + sum_j a[i][j] v[j][c]: 1,024 outputs, 4 a thread
    for (int e = tid; e < LC * LCOLS; e += 256) {
      const int i = e / LCOLS, c = e % LCOLS;
      if (i < n && c < ncols) {
        float o = 0.f;
        for (int d = 0; d < dim; ++d) o = fmaf(qs[i * dq + d], Ss[d * LCOLS + c], o);
        o *= pw[i + 1];
        float w = 0.f;
        for (int j = 0; j <= i; ++j) w = fmaf(as[i * (LC + 1) + j], vs[j * LCOLS + c], w);
        out[(long long)(b0 + i) * heads * vdim + h * vdim + c0 + c] = o + w;
      }
    }
    __syncthreads();
    // S[d][c] = decay^n S[d][c] + sum_j decay^(n-1-j) k_j[d] v_j[c]
    for (int e = tid; e < dim * LCOLS; e += 256) {
      const int d = e / LCOLS, c = e % LCOLS;
      float u = 0.f;
      for (int j = 0; j < n; ++j) u = fmaf(pw[n - 1 - j] * ks[j * dq + d], vs[j * LCOLS + c], u);
      Ss[e] = fmaf(pw[n], Ss[e], u);
    }
  }
  __syncthreads();
  for (int i = tid; i < dim * LCOLS; i += 256) {
    const int d = i / LCOLS, c = i % LCOLS;
    if (c < ncols) S[(long long)d * vdim + c] = Ss[i];
  }
}

extern "C" int jv_lightning_chunk_tokens() { return LC; }
extern "C" int jv_lightning_max_dim(int chunks) { return chunks ? 128 : LT_ROWS * 256; }

#define DEFINE_LIGHTNING(SUF, T)                                                                               \
  extern "C" int jv_lightning_##SUF(float* out, const void* proj, long long ld, int q_off, int k_off,          \
                                    int v_off, float* state, const int* slot_ids, const int* cu_seqlens,       \
                                    const float* decay, int n_requests, int heads, int dim, int vdim,          \
                                    int chunks, void* stream) {                                                \
    if (n_requests <= 0 || heads <= 0) return 0;                                                               \
    if (dim <= 0 || vdim <= 0 || heads > 65535) return (int)hipErrorInvalidValue;                              \
    if (chunks) {                                                                                              \
      if (dim > 128) return (int)hipErrorInvalidValue;                                                         \
      const size_t shmem = (2 * LC * (dim + 1) + LC * LCOLS + LC * (LC + 1) + dim * LCOLS + LC + 1) * sizeof(float); \
      hipLaunchKernelGGL(lightning_chunks_kernel<T>, dim3(n_requests, heads, (vdim + LCOLS - 1) / LCOLS),      \
                         dim3(256), shmem, (hipStream_t)stream, out, (const T*)proj, ld, q_off, k_off, v_off,  \
                         state, slot_ids, cu_seqlens, decay, heads, dim, vdim);                                \
      return JV_LAUNCH_CHECK();                                                                                \
    }                                                                                                          \
    int cols = 64;                       /* the widest slice that keeps a thread's rows in registers */        \
    while (cols > 1 && (cols / 2 >= vdim || (long long)dim * cols > 256LL * LT_ROWS)) cols /= 2;               \
    if ((long long)dim * cols > 256LL * LT_ROWS) return (int)hipErrorInvalidValue;                             \
    const int parts = 256 / cols;                                                                              \
    const size_t shmem = (2 * (2 * dim + cols) + parts * cols) * sizeof(float);                                \
    hipLaunchKernelGGL(lightning_steps_kernel<T>, dim3(n_requests, heads, (vdim + cols - 1) / cols),           \
                       dim3(256), shmem, (hipStream_t)stream, out, (const T*)proj, ld, q_off, k_off, v_off,    \
                       state, slot_ids, cu_seqlens, decay, heads, dim, vdim, cols);                            \
    return JV_LAUNCH_CHECK();                                                                                  \
  }

DEFINE_LIGHTNING(bf16, bf16_t)
DEFINE_LIGHTNING(f32, float)
