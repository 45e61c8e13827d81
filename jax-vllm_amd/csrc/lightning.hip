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
//    so the state is touched once per chunk, a chunk's tokens run side by side, and so do the chunks
//    (everything but the second line's chain).  Only non-negative powers of the decay occur.  Everything is float.
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
// Three launches, so that the chunks of a long prompt run side by side and only the cheap part is serial:
//   local:  per (chunk, head)   a[i][j] = decay^(i-j) q_i . k_j (j <= i);  out_i = sum_j a[i][j] v_j;
//                               U = sum_j decay^(n-1-j) k_j v_j^T                       -> scratch[chunk]
//   scan:   per (request, head) for its chunks in order: scratch[chunk] <- S (the state BEFORE the chunk),
//                               S <- decay^n S + U;  at the end state <- S
//   apply:  per (chunk, head)   out_i += decay^(i+1) S_before^T q_i
#define LC 32        // tokens of a chunk
#define LV 128       // columns (elements of v) a block takes
#define LQ_PAD 4     // row padding of q and k in LDS: rows stay 16-byte aligned

// grid (chunks, heads, column slices of LV); work: chunk -> (request, first token)
template <typename T>
__global__ void __launch_bounds__(256)
lightning_local_kernel(float* __restrict__ out, float* __restrict__ scratch, const T* __restrict__ proj, long long ld,
                       int q_off, int k_off, int v_off, const int* __restrict__ work,
                       const int* __restrict__ cu_seqlens, const float* __restrict__ decay, int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * LV;
  const int r = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(LC, cu_seqlens[r + 1] - b0);
  const int dq = dim + LQ_PAD;
  float* qs = lds;                       // [LC][dq]
  float* ks = qs + LC * dq;              // [LC][dq]
  float* vs = ks + LC * dq;              // [LC][LV]
  float* as = vs + LC * LV;              // [LC][LC + 1]
  float* pw = as + LC * (LC + 1);        // [LC + 1]
  const int tid = threadIdx.x;
  const float lam = decay[h];
  const int ncols = min(LV, vdim - c0);
  if (tid <= LC) pw[tid] = powf(lam, (float)tid);
  for (int i = tid; i < LC * dq; i += 256) {
    const int j = i / dq, d = i - j * dq;
    float qv = 0.f, kv = 0.f;
    if (j < n && d < dim) {
      const T* row = proj + (long long)(b0 + j) * ld;
      qv = lt_silu(to_f32(row[q_off + h * dim + d]));
      kv = lt_silu(to_f32(row[k_off + h * dim + d]));
    }
    qs[i] = qv;
    ks[i] = kv;
  }
  for (int i = tid; i < LC * LV; i += 256) {
    const int j = i / LV, c = i % LV;
    vs[i] = (j < n && c < ncols) ? lt_silu(to_f32(proj[(long long)(b0 + j) * ld + v_off + h * vdim + c0 + c])) : 0.f;
  }
  __syncthreads();
  // a: thread (i, 4 consecutive j)
  {
    const int i = tid >> 3, j0 = (tid & 7) * 4;
    float dot[4] = {0.f, 0.f, 0.f, 0.f};
    if (j0 <= i) {
      for (int d = 0; d < dim; ++d) {
        const float qv = qs[i * dq + d];
#pragma unroll
        for (int u = 0; u < 4; ++u) dot[u] = fmaf(qv, ks[(j0 + u) * dq + d], dot[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) as[i * (LC + 1) + j0 + u] = (j0 + u <= i) ? dot[u] * pw[i - j0 - u] : 0.f;
  }
  __syncthreads();
  // k_j <- decay^(n-1-j) k_j (rows beyond the chunk are zero already); out = a v
  for (int i = tid; i < LC * dq; i += 256) {
    const int j = i / dq;
    if (j < n) ks[i] *= pw[n - 1 - j];
  }
  for (int e = tid; e < LC * (LV / 4); e += 256) {
    const int i = e / (LV / 4), c = (e % (LV / 4)) * 4;
    if (i < n && c < ncols) {
      float4 o = {0.f, 0.f, 0.f, 0.f};
      for (int j = 0; j <= i; ++j) {
        const float a = as[i * (LC + 1) + j];
        const float4 v = *(const float4*)(vs + j * LV + c);
        o.x = fmaf(a, v.x, o.x); o.y = fmaf(a, v.y, o.y); o.z = fmaf(a, v.z, o.z); o.w = fmaf(a, v.w, o.w);
      }
      float* dst = out + (long long)(b0 + i) * heads * vdim + h * vdim + c0 + c;
      dst[0] = o.x;
      if (c + 1 < ncols) dst[1] = o.y;
      if (c + 2 < ncols) dst[2] = o.z;
      if (c + 3 < ncols) dst[3] = o.w;
    }
  }
  __syncthreads();
  // U[d][c]: tiles of 4 x 4 per thread
  float* U = scratch + (((long long)ch * heads + h) * dim) * vdim + c0;
  const int dt = (dim + 3) / 4;
  for (int e = tid; e < dt * (LV / 4); e += 256) {
    const int d0 = (e / (LV / 4)) * 4, c = (e % (LV / 4)) * 4;
    if (c >= ncols) continue;
    float u[4][4] = {};
    for (int j = 0; j < n; ++j) {
      const float4 kv = *(const float4*)(ks + j * dq + d0);
      const float4 v = *(const float4*)(vs + j * LV + c);
      const float kk[4] = {kv.x, kv.y, kv.z, kv.w}, vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) u[a][b] = fmaf(kk[a], vv[b], u[a][b]);
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (d0 + a < dim)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          if (c + b < ncols) U[(long long)(d0 + a) * vdim + c + b] = u[a][b];
  }
}

// grid (requests, heads, slices of the dim x vdim elements); req_chunks [requests + 1]: first chunk of each request
__global__ void __launch_bounds__(256)
lightning_scan_kernel(float* __restrict__ scratch, float* __restrict__ state, const int* __restrict__ slot_ids,
                      const int* __restrict__ req_chunks, const int* __restrict__ work,
                      const int* __restrict__ cu_seqlens, const float* __restrict__ decay, int heads, int dim, int vdim) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int first = req_chunks[r], last = req_chunks[r + 1];
  if (last <= first) return;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= dim * vdim) return;
  const float lam = decay[h];
  float* S = state + ((long long)slot_ids[r] * heads + h) * dim * vdim + e;
  float s = *S;
  const int end = cu_seqlens[r + 1];
  float next = scratch[((long long)first * heads + h) * dim * vdim + e];
  for (int ch = first; ch < last; ++ch) {
    float* U = scratch + ((long long)ch * heads + h) * dim * vdim + e;
    const float u = next;
    if (ch + 1 < last) next = U[(long long)heads * dim * vdim];     // asked for before this chunk's store
    *U = s;
    const int n = min(LC, end - work[2 * ch + 1]);
    s = fmaf(powf(lam, (float)n), s, u);
  }
  *S = s;
}

// grid as the local kernel
template <typename T>
__global__ void __launch_bounds__(256)
lightning_apply_kernel(float* __restrict__ out, const float* __restrict__ scratch, const T* __restrict__ proj,
                       long long ld, int q_off, const int* __restrict__ work, const int* __restrict__ cu_seqlens,
                       const float* __restrict__ decay, int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * LV;
  const int r = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(LC, cu_seqlens[r + 1] - b0);
  const int dq = dim + 1;
  float* qs = lds;                       // [LC][dq]
  float* ps = qs + LC * dq;              // [32][LV]: a slab of 32 rows of the state
  const int tid = threadIdx.x;
  const int ncols = min(LV, vdim - c0);
  for (int i = tid; i < LC * dim; i += 256) {
    const int j = i / dim, d = i - j * dim;
    qs[j * dq + d] = j < n ? lt_silu(to_f32(proj[(long long)(b0 + j) * ld + q_off + h * dim + d])) : 0.f;
  }
  const float* P = scratch + (((long long)ch * heads + h) * dim) * vdim + c0;
  const int i0 = (tid >> 5) * 4, c = (tid & 31) * 4;       // thread: rows i0..i0+3, columns c..c+3
  float o[4][4] = {};
  for (int d0 = 0; d0 < dim; d0 += 32) {
    __syncthreads();
    for (int e = tid; e < 32 * LV; e += 256) {
      const int d = d0 + e / LV, cc = e % LV;
      ps[e] = (d < dim && cc < ncols) ? P[(long long)d * vdim + cc] : 0.f;
    }
    __syncthreads();
    const int dn = min(32, dim - d0);
    for (int d = 0; d < dn; ++d) {
      const float4 p = *(const float4*)(ps + d * LV + c);
      const float pp[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const float qv = qs[(i0 + a) * dq + d0 + d];
#pragma unroll
        for (int b = 0; b < 4; ++b) o[a][b] = fmaf(qv, pp[b], o[a][b]);
      }
    }
  }
  const float lam = decay[h];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int i = i0 + a;
    if (i >= n) continue;
    const float w = powf(lam, (float)(i + 1));
    float* dst = out + (long long)(b0 + i) * heads * vdim + h * vdim + c0 + c;
#pragma unroll
    for (int b = 0; b < 4; ++b)
      if (c + b < ncols) dst[b] += w * o[a][b];
  }
}

extern "C" int jv_lightning_chunk_tokens() { return LC; }
extern "C" int jv_lightning_max_dim(int chunks) { return chunks ? 128 : LT_ROWS * 256; }

// chunks = 0: token by token.  chunks = number of chunks (> 0): by chunks, with work [chunks][2] = (request,
// first token) in the order of requests and tokens, req_chunks [requests + 1], and scratch of
// chunks * heads * dim * vdim floats.
#define DEFINE_LIGHTNING(SUF, T)                                                                               \
  extern "C" int jv_lightning_##SUF(float* out, const void* proj, long long ld, int q_off, int k_off,          \
                                    int v_off, float* state, const int* slot_ids, const int* cu_seqlens,       \
                                    const float* decay, int n_requests, int heads, int dim, int vdim,          \
                                    int chunks, const int* work, const int* req_chunks, float* scratch,        \
                                    void* stream) {                                                            \
    if (n_requests <= 0 || heads <= 0) return 0;                                                               \
    if (dim <= 0 || vdim <= 0 || heads > 65535) return (int)hipErrorInvalidValue;                              \
    hipStream_t s = (hipStream_t)stream;                                                                       \
    if (chunks > 0) {                                                                                          \
      if (dim > 128 || !work || !req_chunks || !scratch) return (int)hipErrorInvalidValue;                     \
      const int slices = (vdim + LV - 1) / LV;                                                                 \
      const size_t lds_local = (2 * LC * (dim + LQ_PAD) + LC * LV + LC * (LC + 1) + LC + 1) * sizeof(float);   \
      const size_t lds_apply = (LC * (dim + 1) + 32 * LV) * sizeof(float);                                     \
      hipLaunchKernelGGL(lightning_local_kernel<T>, dim3(chunks, heads, slices), dim3(256), lds_local, s, out, \
                         scratch, (const T*)proj, ld, q_off, k_off, v_off, work, cu_seqlens, decay, heads,     \
                         dim, vdim);                                                                           \
      hipLaunchKernelGGL(lightning_scan_kernel, dim3(n_requests, heads, (dim * vdim + 255) / 256), dim3(256),  \
                         0, s, scratch, state, slot_ids, req_chunks, work, cu_seqlens, decay, heads, dim,      \
                         vdim);                                                                                \
      hipLaunchKernelGGL(lightning_apply_kernel<T>, dim3(chunks, heads, slices), dim3(256), lds_apply, s, out, \
                         scratch, (const T*)proj, ld, q_off, work, cu_seqlens, decay, heads, dim, vdim);       \
      return JV_LAUNCH_CHECK();                                                                                \
    }                                                                                                          \
    int cols = 64;                       /* the widest slice that keeps a thread's rows in registers */        \
    while (cols > 1 && (cols / 2 >= vdim || (long long)dim * cols > 256LL * LT_ROWS)) cols /= 2;               \
    if ((long long)dim * cols > 256LL * LT_ROWS) return (int)hipErrorInvalidValue;                             \
    const int parts = 256 / cols;                                                                              \
    const size_t shmem = (2 * (2 * dim + cols) + parts * cols) * sizeof(float);                                \
    hipLaunchKernelGGL(lightning_steps_kernel<T>, dim3(n_requests, heads, (vdim + cols - 1) / cols),           \
                       dim3(256), shmem, s, out, (const T*)proj, ld, q_off, k_off, v_off,                      \
                       state, slot_ids, cu_seqlens, decay, heads, dim, vdim, cols);                            \
    return JV_LAUNCH_CHECK();                                                                                  \
  }

DEFINE_LIGHTNING(bf16, bf16_t)
DEFINE_LIGHTNING(f32, float)
