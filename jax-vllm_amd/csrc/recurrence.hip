// Recurrent mixers with a float matrix state per request and head, and what stands around them:
//
//   short_conv        a causal convolution over time per channel whose last taps - 1 inputs are state
//   recurrence_gates  per (token, head): decay g = exp(-exp(A) softplus(raw + bias)) and a write strength
//                     (the step size itself, or sigmoid of another column)
//   heads_to_f32      heads of a projection as float, optionally rotated by position and scaled
//   head_unit_norm    x / sqrt(sum(x^2) + eps) * scale per head, in place on the leading heads of every row
//   recurrence_steps  S <- g S;  u = w (v - [delta] S^T k);  S <- S + k u^T;  o = S^T q (+ skip v)
//   group_gated_norm  norm of float rows in equal groups, a gate before or behind it
//
// One recurrence serves retention (g constant per head, w = 1), the state-space form (k and q shared by a
// group of heads, w = step size, skip) and the gated delta rule (delta = 1, w = beta).  Everything that
// enters it is float.  The state of a request lives in a row of `state` [slots + 1][heads][dim][vdim]
// between steps.  Columns of S never mix, so a block takes one (request, head, slice of columns) and a
// thread keeps up to RC_ROWS rows of one column in registers.
#include "common.h"

#define RC_ROWS 32
#define RC_MAX_LAGS 7        // a convolution has at most 8 taps

__device__ __forceinline__ float rc_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float rc_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------- short causal convolution with state
// out[t][c] = act( bias[c] + sum_j w[c][j] * in[t - (taps - 1) + j][c] ), in = proj[:, c_off + c] of the
// request's tokens, continued to the left by the request's state rows [taps - 1][channels] (lag taps - 1
// first).  grid (requests, channel blocks, segments of seg_len tokens); the thread of segment 0 also
// writes the state the step leaves (it is the only one that reads the old one).
template <typename T>
__global__ void __launch_bounds__(256)
short_conv_kernel(float* __restrict__ out, long long ldo, const T* __restrict__ proj, long long ld, int c_off,
                  int channels, int taps, const float* __restrict__ w, const float* __restrict__ bias,
                  float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_seqlens,
                  int act, int seg_len) {
  const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int t0 = cu_seqlens[r], n = cu_seqlens[r + 1] - t0;
  const int s0 = blockIdx.z * seg_len;
  if (s0 >= n) return;
  const int lags = taps - 1;
  float* st = state + (long long)slot_ids[r] * lags * channels + c;
  const T* in = proj + (long long)t0 * ld + c_off + c;
  // slot p of the window holds the input of lag RC_MAX_LAGS - p; lags the filter does not have weigh nothing
  float win[RC_MAX_LAGS], wl[RC_MAX_LAGS];
#pragma unroll
  for (int p = 0; p < RC_MAX_LAGS; ++p) {
    const int lag = RC_MAX_LAGS - p;
    float x = 0.f, f = 0.f;
    if (lag <= lags) {
      f = w[(long long)c * taps + lags - lag];
      const int i = s0 - lag;
      x = i >= 0 ? to_f32(in[(long long)i * ld]) : st[(long long)(lags + i) * channels];
    }
    win[p] = x;
    wl[p] = f;
  }
  const float w0 = w[(long long)c * taps + lags], b = bias ? bias[c] : 0.f;
  const int s1 = min(n, s0 + seg_len);
  for (int i = s0; i < s1; ++i) {
    const float x = to_f32(in[(long long)i * ld]);
    float acc = b;
#pragma unroll
    for (int p = 0; p < RC_MAX_LAGS; ++p) acc = fmaf(wl[p], win[p], acc);
    acc = fmaf(w0, x, acc);
    out[(long long)(t0 + i) * ldo + c] = act ? rc_silu(acc) : acc;
#pragma unroll
    for (int p = 0; p + 1 < RC_MAX_LAGS; ++p) win[p] = win[p + 1];
    win[RC_MAX_LAGS - 1] = x;
  }
  if (blockIdx.z == 0) {
    // the last `lags` inputs of the request: rows of this step, or, for a short step, old state rows moved up
    // (row j takes row j + n: read before any row above j is written)
    for (int j = 0; j < lags; ++j) {
      const int i = n - lags + j;
      st[(long long)j * channels] = i >= 0 ? to_f32(in[(long long)i * ld]) : st[(long long)(j + n) * channels];
    }
  }
}

// ---------------------------------------------------------------- decays and write strengths
// mode 0: dt = softplus(raw + bias);  g = exp(-exp(A) dt);  w = dt
// mode 1: g as above from the column at dt_off;  w = sigmoid(column at w_off)
template <typename T>
__global__ void __launch_bounds__(256)
recurrence_gates_kernel(float* __restrict__ g, float* __restrict__ wgt, const T* __restrict__ proj, long long ld,
                        int dt_off, int w_off, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                        int n, int heads, int mode) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long long)n * heads) return;
  const int t = (int)(e / heads), h = (int)(e % heads);
  const float dt = rc_softplus(to_f32(proj[(long long)t * ld + dt_off + h]) + dt_bias[h]);
  g[e] = expf(-expf(a_log[h]) * dt);
  wgt[e] = mode == 0 ? dt : 1.f / (1.f + expf(-to_f32(proj[(long long)t * ld + w_off + h])));
}

// ---------------------------------------------------------------- heads as float, rotated and scaled
// out[t][h][i] of `width` = heads * d columns of proj from `off`; the first rot_dims elements of a head turn
// by the token's angles (cos_sin [n][rot_dims]: cosines, then sines; element i pairs with i + rot_dims / 2).
template <typename T>
__global__ void __launch_bounds__(256)
heads_to_f32_kernel(float* __restrict__ out, const T* __restrict__ proj, long long ld, int off, int n, int heads,
                    int d, int rot_dims, const float* __restrict__ cos_sin, float scale) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  const int width = heads * d;
  if (e >= (long long)n * width) return;
  const int t = (int)(e / width), c = (int)(e % width), i = c % d;
  const T* row = proj + (long long)t * ld + off;
  float x = to_f32(row[c]);
  if (i < rot_dims) {
    const int half = rot_dims / 2, j = i < half ? i : i - half;
    const float cs = cos_sin[(long long)t * rot_dims + j], sn = cos_sin[(long long)t * rot_dims + half + j];
    const float other = to_f32(row[i < half ? c + half : c - half]);
    x = i < half ? x * cs - other * sn : x * cs + other * sn;
  }
  out[e] = x * scale;
}

// The same for q, k and v of one mixer at once: proj rows [q: heads * d | k: heads * d | v: heads * dv | ...] become float
// rows [q | k | v]; q and k turn by position, k is multiplied by k_scale, v is copied.
template <typename T>
__global__ void __launch_bounds__(256)
qkv_to_f32_kernel(float* __restrict__ out, const T* __restrict__ proj, long long ld, int n, int heads, int d, int dv,
                  int rot_dims, const float* __restrict__ cos_sin, float k_scale) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  const int qk = heads * d, width = 2 * qk + heads * dv;
  if (e >= (long long)n * width) return;
  const int t = (int)(e / width), c = (int)(e % width);
  const T* row = proj + (long long)t * ld;
  float x = to_f32(row[c]);
  if (c < 2 * qk) {
    const int i = c % d;
    if (i < rot_dims) {
      const int half = rot_dims / 2, j = i < half ? i : i - half;
      const float cs = cos_sin[(long long)t * rot_dims + j], sn = cos_sin[(long long)t * rot_dims + half + j];
      const float other = to_f32(row[i < half ? c + half : c - half]);
      x = i < half ? x * cs - other * sn : x * cs + other * sn;
    }
    if (c >= qk) x *= k_scale;
  }
  out[e] = x;
}

// x [n][ld] float, in place on the first `heads` runs of d columns of every row: x / sqrt(sum(x^2) + eps) * scale,
// scale = scale_a for the first `heads_a` heads of a row and scale_b for the others; one wave a head
__global__ void __launch_bounds__(256)
head_unit_norm_kernel(float* __restrict__ x, long long ld, long long n, int heads, int d, float eps, int heads_a,
                      float scale_a, float scale_b) {
  const long long r = (long long)blockIdx.x * 4 + threadIdx.x / JV_WAVE;
  if (r >= n * heads) return;
  const int lane = threadIdx.x % JV_WAVE;
  const int hd = (int)(r % heads);
  float* p = x + (r / heads) * ld + (long long)hd * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += JV_WAVE) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float inv = (hd < heads_a ? scale_a : scale_b) / sqrtf(ss + eps);
  for (int i = lane; i < d; i += JV_WAVE) p[i] *= inv;
}

// ---------------------------------------------------------------- the recurrence, token by token
// grid (requests, heads, column slices); block 256 = parts x cols threads, cols a power of two.
// q, k: [n][qk_heads][dim] (row strides ldq, ldk), head h reads qk head h / (heads / qk_heads);
// v: [n][heads][vdim]; g: [n][heads] (g_stride = heads) or [heads] (g_stride = 0); wgt [n][heads] or null (1);
// skip [heads] or null: out += skip[h] * v.
__global__ void __launch_bounds__(256)
recurrence_steps_kernel(float* __restrict__ out, const float* __restrict__ q, long long ldq,
                        const float* __restrict__ k, long long ldk, const float* __restrict__ v, long long ldv,
                        const float* __restrict__ g, int g_stride, const float* __restrict__ wgt,
                        const float* __restrict__ skip, float* __restrict__ state, const int* __restrict__ slot_ids,
                        const int* __restrict__ cu_seqlens, int heads, int qk_heads, int dim, int vdim, int cols,
                        int delta) {
  extern __shared__ float lds[];          // 2 x (q[dim] | k[dim] | v[cols]) | two arrays of partial sums [parts][cols]
  const int r = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * cols;
  const int parts = blockDim.x / cols;
  const int col = threadIdx.x % cols, part = threadIdx.x / cols;
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  if (t1 <= t0) return;
  const int stage = 2 * dim + cols;
  float* red_a = lds + 2 * stage;
  float* red_b = red_a + parts * cols;
  const int hk = h / (heads / qk_heads);
  const bool live = c0 + col < vdim;
  const float sk = skip ? skip[h] : 0.f;
  float* S = state + (((long long)slot_ids[r] * heads + h) * dim) * vdim + c0 + col;
  float s[RC_ROWS];
#pragma unroll
  for (int i = 0; i < RC_ROWS; ++i) {
    const int d = part + i * parts;
    s[i] = (live && d < dim) ? S[(long long)d * vdim] : 0.f;
  }
  for (int t = t0; t < t1; ++t) {
    float* buf = lds + ((t - t0) & 1) * stage;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
      buf[d] = q[(long long)t * ldq + hk * dim + d];
      buf[dim + d] = k[(long long)t * ldk + hk * dim + d];
    }
    if (threadIdx.x < cols)
      buf[2 * dim + threadIdx.x] = (c0 + threadIdx.x < vdim) ? v[(long long)t * ldv + h * vdim + c0 + threadIdx.x] : 0.f;
    const float gt = g[(long long)t * g_stride + h];
    const float wt = wgt ? wgt[(long long)t * heads + h] : 1.f;
    __syncthreads();
    const float vv = buf[2 * dim + col];
    float u = wt * vv;
    if (delta) {
      float pred = 0.f;
#pragma unroll
      for (int i = 0; i < RC_ROWS; ++i) {
        const int d = part + i * parts;
        if (d < dim) {
          s[i] *= gt;
          pred = fmaf(s[i], buf[dim + d], pred);
        }
      }
      red_a[part * cols + col] = pred;
      __syncthreads();
      pred = 0.f;
      for (int p = 0; p < parts; ++p) pred += red_a[p * cols + col];
      u = wt * (vv - pred);
    }
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < RC_ROWS; ++i) {
      const int d = part + i * parts;
      if (d < dim) {
        s[i] = delta ? fmaf(buf[dim + d], u, s[i]) : fmaf(gt, s[i], buf[dim + d] * u);
        acc = fmaf(s[i], buf[d], acc);
      }
    }
    red_b[part * cols + col] = acc;
    __syncthreads();
    if (part == 0 && live) {
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += red_b[p * cols + col];
      out[(long long)t * heads * vdim + h * vdim + c0 + col] = fmaf(sk, vv, o);
    }
    // the next token fills the other stage; red_a and red_b are rewritten only behind the barrier after that fill
  }
#pragma unroll
  for (int i = 0; i < RC_ROWS; ++i) {
    const int d = part + i * parts;
    if (live && d < dim) S[(long long)d * vdim] = s[i];
  }
}

// ---------------------------------------------------------------- the recurrence by chunks (delta = 0)
// With c_i = sum_{m <= i} log g_m inside a chunk of n <= RC_LC tokens and S0 the state before it:
//     o_i   = exp(c_i) S0^T q_i + sum_{j <= i} exp(c_i - c_j) (q_i . k_j) w_j v_j  (+ skip v_i)
//     S_end = exp(c_(n-1)) S0 + sum_j exp(c_(n-1) - c_j) w_j k_j v_j^T
// Only differences c_i - c_j <= 0 are exponentiated (a decay of 0 counts as 1e-38).  Three launches, so that the
// chunks of a long prompt run side by side and only the cheap part is serial:
//   local:  per (chunk, head, slice)  out_i = sum_j a[i][j] v_j;  U = sum_j k'_j v_j^T -> scratch[chunk];  exp(c_i) -> cum
//   scan:   per (request, head)       for its chunks in order: scratch[chunk] <- S (the state BEFORE the chunk),
//                                     S <- exp(c_(n-1)) S + U;  at the end state <- S
//   apply:  per (chunk, head, slice)  out_i += exp(c_i) S_before^T q_i
#define RC_LC 32        // tokens of a chunk
#define RC_LV 128       // columns (elements of v) a block takes
#define RC_PAD 4        // row padding of q and k in LDS: rows stay 16-byte aligned

// grid (chunks, heads, column slices of RC_LV); work: chunk -> (request, first token).  The three products run on the
// matrix cores in true 32-bit (v_mfma_f32_32x32x2_f32): the scores q_i . k_j with the key size shared out to the four
// waves, then per wave 32 of the block's columns: out = a V and U = K'^T V from the same operands of V, which come
// straight from global memory (every element is used by one wave only).
typedef float rc_f32x16 __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256)
recurrence_local_kernel(float* __restrict__ out, float* __restrict__ scratch, float* __restrict__ cum,
                        const float* __restrict__ q, long long ldq, const float* __restrict__ k, long long ldk,
                        const float* __restrict__ v, long long ldv, const float* __restrict__ g, int g_stride,
                        const float* __restrict__ wgt, const float* __restrict__ skip, const int* __restrict__ work,
                        const int* __restrict__ cu_seqlens, int heads, int qk_heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * RC_LV;
  const int r = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(RC_LC, cu_seqlens[r + 1] - b0);
  const int hk = h / (heads / qk_heads);
  const int dq = dim + 1, lm = RC_LC + 1;
  float* qs = lds;                       // [LC][dq]
  float* ks = qs + RC_LC * dq;           // [LC][dq]
  float* ps = ks + RC_LC * dq;           // [4][LC][LC + 1]: the waves' shares of the scores
  float* as = ps + 4 * RC_LC * lm;       // [LC][LC + 1]
  float* cl = as + RC_LC * lm;           // [LC] cumulative log decay
  float* ws = cl + RC_LC;                // [LC] write strengths
  const int tid = threadIdx.x;
  const int wave = tid / JV_WAVE, lane = tid % JV_WAVE, col = lane % 32, kh = lane / 32;
  if (tid < RC_LC) {
    float lg = 0.f, w = 0.f;
    if (tid < n) {
      lg = logf(fmaxf(g[(long long)(b0 + tid) * g_stride + h], 1e-38f));
      w = wgt ? wgt[(long long)(b0 + tid) * heads + h] : 1.f;
    }
    // inclusive prefix sum over the first 32 lanes of wave 0
#pragma unroll
    for (int o = 1; o < RC_LC; o <<= 1) {
      const float up = __shfl_up(lg, o, JV_WAVE);
      if (tid >= o) lg += up;
    }
    cl[tid] = lg;
    ws[tid] = w;
    if (blockIdx.z == 0 && tid < n) cum[(long long)(b0 + tid) * heads + h] = expf(lg);
  }
  for (int i = tid; i < RC_LC * dim; i += 256) {
    const int j = i / dim, d = i - j * dim;
    float qv = 0.f, kv = 0.f;
    if (j < n) {
      qv = q[(long long)(b0 + j) * ldq + hk * dim + d];
      kv = k[(long long)(b0 + j) * ldk + hk * dim + d];
    }
    qs[j * dq + d] = qv;
    ks[j * dq + d] = kv;
  }
  __syncthreads();
  {  // scores: wave w sums over its quarter of the key elements, two a product (one a half wave)
    const int share = dim / 4, d0 = wave * share;          // dim is a multiple of 4; a share may be odd
    rc_f32x16 acc = {};
    for (int d = 0; d < share; d += 2) {
      const int dd = d0 + d + kh;
      const bool in = d + kh < share;
      const float a = in ? qs[col * dq + dd] : 0.f, bq = in ? ks[col * dq + dd] : 0.f;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bq, acc, 0, 0, 0);
    }
    float* mine = ps + wave * RC_LC * lm;
#pragma unroll
    for (int e = 0; e < 16; ++e) mine[((e / 4) * 8 + kh * 4 + e % 4) * lm + col] = acc[e];
  }
  __syncthreads();
  {  // a[i][j] = (q_i . k_j) exp(c_i - c_j) w_j (+ skip on the diagonal): thread (i, 4 consecutive j)
    const int i = tid >> 3, j0 = (tid & 7) * 4;
    const float sk = skip ? skip[h] : 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u;
      float a = 0.f;
      if (j <= i && i < n) {
        const float dot = (ps[i * lm + j] + ps[(RC_LC + i) * lm + j]) + (ps[(2 * RC_LC + i) * lm + j] + ps[(3 * RC_LC + i) * lm + j]);
        a = dot * expf(cl[i] - cl[j]) * ws[j] + (j == i ? sk : 0.f);
      }
      as[i * lm + j] = a;
    }
  }
  // k_j <- exp(c_(n-1) - c_j) w_j k_j (rows beyond the chunk are zero already)
  for (int i = tid; i < RC_LC * dim; i += 256) {
    const int j = i / dim, d = i - j * dim;
    if (j < n) ks[j * dq + d] *= expf(cl[n - 1] - cl[j]) * ws[j];
  }
  __syncthreads();
  const int wc0 = c0 + wave * 32;                          // this wave's first column
  if (wc0 >= vdim) return;
  const bool live = wc0 + col < vdim;
  const float* V = v + (long long)b0 * ldv + h * vdim + wc0 + (live ? col : 0);
  const int tiles = (dim + 31) / 32;                       // row tiles of U, at most 4
  rc_f32x16 o = {}, u0 = {}, u1 = {}, u2 = {}, u3 = {};
  for (int j = 0; j < RC_LC; j += 2) {
    const int jj = j + kh;
    const float vv = V[(long long)min(jj, n - 1) * ldv];
    const float bv = (live && jj < n) ? vv : 0.f;
    o = __builtin_amdgcn_mfma_f32_32x32x2f32(as[col * lm + jj], bv, o, 0, 0, 0);
    const float* kr = ks + jj * dq + col;                  // K'^T: row d = 32 t + col, column jj
    u0 = __builtin_amdgcn_mfma_f32_32x32x2f32(kr[0], bv, u0, 0, 0, 0);
    if (tiles > 1) u1 = __builtin_amdgcn_mfma_f32_32x32x2f32(col + 32 < dim ? kr[32] : 0.f, bv, u1, 0, 0, 0);
    if (tiles > 2) u2 = __builtin_amdgcn_mfma_f32_32x32x2f32(col + 64 < dim ? kr[64] : 0.f, bv, u2, 0, 0, 0);
    if (tiles > 3) u3 = __builtin_amdgcn_mfma_f32_32x32x2f32(col + 96 < dim ? kr[96] : 0.f, bv, u3, 0, 0, 0);
  }
  if (!live) return;
  float* U = scratch + (((long long)ch * heads + h) * dim) * vdim + wc0 + col;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int i = (e / 4) * 8 + kh * 4 + e % 4;            // the row of accumulator element e
    if (i < n) out[(long long)(b0 + i) * heads * vdim + h * vdim + wc0 + col] = o[e];
    if (i < dim) U[(long long)i * vdim] = u0[e];
    if (i + 32 < dim) U[(long long)(i + 32) * vdim] = u1[e];
    if (i + 64 < dim) U[(long long)(i + 64) * vdim] = u2[e];
    if (i + 96 < dim) U[(long long)(i + 96) * vdim] = u3[e];
  }
}

// grid (requests, heads, slices of the dim x vdim elements); req_chunks [requests + 1]: first chunk of each request
__global__ void __launch_bounds__(256)
recurrence_scan_kernel(float* __restrict__ scratch, float* __restrict__ state, const float* __restrict__ cum,
                       const int* __restrict__ slot_ids, const int* __restrict__ req_chunks,
                       const int* __restrict__ work, const int* __restrict__ cu_seqlens, int heads, int dim, int vdim) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int first = req_chunks[r], last = req_chunks[r + 1];
  if (last <= first) return;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= dim * vdim) return;
  float* S = state + ((long long)slot_ids[r] * heads + h) * dim * vdim + e;
  float s = *S;
  const int end = cu_seqlens[r + 1];
  float next = scratch[((long long)first * heads + h) * dim * vdim + e];
  for (int ch = first; ch < last; ++ch) {
    float* U = scratch + ((long long)ch * heads + h) * dim * vdim + e;
    const float u = next;
    if (ch + 1 < last) next = U[(long long)heads * dim * vdim];     // asked for before this chunk's store
    *U = s;
    const int b0 = work[2 * ch + 1];
    const int n = min(RC_LC, end - b0);
    s = fmaf(cum[(long long)(b0 + n - 1) * heads + h], s, u);
  }
  *S = s;
}

// grid as the local kernel.  out[32 x LV] += diag(cum) Q[32 x dim] P[dim x LV] on the matrix cores in true 32-bit
// (v_mfma_f32_32x32x2_f32: float operands, float products and sums): a wave takes 32 of the block's columns, its B
// operands come straight from the state in global memory (every element is used by one wave only), A from LDS.
__global__ void __launch_bounds__(256)
recurrence_apply_kernel(float* __restrict__ out, const float* __restrict__ scratch, const float* __restrict__ cum,
                        const float* __restrict__ q, long long ldq, const int* __restrict__ work,
                        const int* __restrict__ cu_seqlens, int heads, int qk_heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * RC_LV;
  const int r = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(RC_LC, cu_seqlens[r + 1] - b0);
  const int hk = h / (heads / qk_heads);
  const int dq = dim + 1;
  float* qs = lds;                       // [LC][dq]
  const int tid = threadIdx.x;
  for (int i = tid; i < RC_LC * dim; i += 256) {
    const int j = i / dim, d = i - j * dim;
    qs[j * dq + d] = j < n ? q[(long long)(b0 + j) * ldq + hk * dim + d] : 0.f;
  }
  __syncthreads();
  const int wave = tid / JV_WAVE, lane = tid % JV_WAVE;
  const int wc0 = c0 + wave * 32;                          // this wave's first column
  if (wc0 >= vdim) return;
  const int col = lane % 32, kh = lane / 32;
  const bool live = wc0 + col < vdim;
  const float* P = scratch + (((long long)ch * heads + h) * dim) * vdim + wc0 + (live ? col : 0);
  const float* A = qs + col * dq + kh;                     // row `col` of Q, elements kh, kh + 2, ...
  rc_f32x16 acc = {};
  // two products a turn (dim is a multiple of 4), their loads asked for together
  for (int d = 0; d < dim; d += 4) {
    const float b0v = P[(long long)(d + kh) * vdim], b1v = P[(long long)(d + 2 + kh) * vdim];
    const float a0 = A[d], a1 = A[d + 2];
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, live ? b0v : 0.f, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, live ? b1v : 0.f, acc, 0, 0, 0);
  }
  if (!live) return;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int i = (e / 4) * 8 + kh * 4 + e % 4;            // the row of accumulator element e
    if (i < n) {
      const float w = cum ? cum[(long long)(b0 + i) * heads + h] : 1.f;
      out[(long long)(b0 + i) * heads * vdim + h * vdim + wc0 + col] += w * acc[e];
    }
  }
}

extern "C" int jv_recurrence_chunk_tokens() { return RC_LC; }
extern "C" int jv_recurrence_chunk_max_dim() { return 128; }

// work [chunks][2] = (request, first token) in the order of requests and tokens, req_chunks [requests + 1], scratch of
// chunks * heads * dim * vdim floats, cum of tokens * heads floats.
extern "C" int jv_recurrence_chunks(float* out, const float* q, long long ldq, const float* k, long long ldk,
                                    const float* v, long long ldv, const float* g, int g_stride, const float* wgt,
                                    const float* skip, float* state, const int* slot_ids, const int* cu_seqlens,
                                    int n_requests, int heads, int qk_heads, int dim, int vdim, int chunks,
                                    const int* work, const int* req_chunks, float* scratch, float* cum, void* stream) {
  if (n_requests <= 0 || heads <= 0 || chunks <= 0) return 0;
  if (dim <= 0 || dim > 128 || dim % 4 || vdim <= 0 || heads > 65535 || qk_heads <= 0 || heads % qk_heads || !work ||
      !req_chunks || !scratch || !cum)
    return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  const int slices = (vdim + RC_LV - 1) / RC_LV;
  const size_t lds_local = (2 * RC_LC * (dim + 1) + 5 * RC_LC * (RC_LC + 1) + 2 * RC_LC) * sizeof(float);
  const size_t lds_apply = (size_t)RC_LC * (dim + 1) * sizeof(float);
  hipLaunchKernelGGL(recurrence_local_kernel, dim3(chunks, heads, slices), dim3(256), lds_local, s, out, scratch, cum, q,
                     ldq, k, ldk, v, ldv, g, g_stride, wgt, skip, work, cu_seqlens, heads, qk_heads, dim, vdim);
  hipLaunchKernelGGL(recurrence_scan_kernel, dim3(n_requests, heads, (dim * vdim + 255) / 256), dim3(256), 0, s, scratch,
                     state, cum, slot_ids, req_chunks, work, cu_seqlens, heads, dim, vdim);
  hipLaunchKernelGGL(recurrence_apply_kernel, dim3(chunks, heads, slices), dim3(256), lds_apply, s, out, scratch, cum, q,
                     ldq, work, cu_seqlens, heads, qk_heads, dim, vdim);
  return JV_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- the delta rule by chunks
// Inside a chunk (c_i as above, G_i = exp(c_i), beta_i the write strength, S0 the state before it) the updates
//     u_i = beta_i (v_i - (g_i S_(i-1))^T k_i),   S_i = g_i S_(i-1) + k_i u_i^T
// obey  u_i = beta_i (v_i - G_i S0^T k_i - sum_{j<i} A_ij u_j),  A_ij = exp(c_i - c_j) (k_i . k_j), so with the lower
// triangular T = (I + diag(beta) A)^-1 diag(beta):
//     U = Wv - Wk S0,             Wv = T V,  Wk = T diag(G) K
//     O = Qt S0 + (B T) V,        B_ij = exp(c_i - c_j) (q_i . k_j) (j <= i),  Qt = diag(G) Q - (B T) diag(G) K
//     S_end = G_(n-1) S0 + Kd^T U,   Kd_j = exp(c_(n-1) - c_j) k_j
// Three launches: `local` makes T, Wk, Kd, Qt, Wv and the chunk-local outputs (B T) V for all chunks side by side;
// `scan` walks a request's chunks in order with a slice of S in LDS (two small products a chunk) and leaves the state
// before every chunk in scratch; the plain recurrence's `apply` adds Qt S_before.
// grid (chunks, heads)
__global__ void __launch_bounds__(256)
delta_local_kernel(float* __restrict__ out, float* __restrict__ wk_out, float* __restrict__ kd_out,
                   float* __restrict__ wv_out, float* __restrict__ qt_out, float* __restrict__ cum,
                   const float* __restrict__ q, long long ldq, const float* __restrict__ k, long long ldk,
                   const float* __restrict__ v, long long ldv, const float* __restrict__ g, int g_stride,
                   const float* __restrict__ wgt, const int* __restrict__ work, const int* __restrict__ cu_seqlens,
                   int heads, int qk_heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int ch = blockIdx.x, h = blockIdx.y;
  const int r = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(RC_LC, cu_seqlens[r + 1] - b0);
  const int hk = h / (heads / qk_heads);
  const int dq = dim + RC_PAD, lm = RC_LC + 1;
  float* qs = lds;                       // [LC][dq]
  float* ks = qs + RC_LC * dq;           // [LC][dq]
  float* ma = ks + RC_LC * dq;           // [LC][LC + 1]: A, later B T
  float* mb = ma + RC_LC * lm;           // [LC][LC + 1]: B
  float* mt = mb + RC_LC * lm;           // [LC][LC + 1]: T
  float* vs = mt + RC_LC * lm;           // [LC][LV]
  float* cl = vs + RC_LC * RC_LV;        // [LC] cumulative log decay
  float* bs = cl + RC_LC;                // [LC] beta
  float* gs = bs + RC_LC;                // [LC] exp(cl)
  const int tid = threadIdx.x;
  if (tid < RC_LC) {
    float lg = 0.f, w = 0.f;
    if (tid < n) {
      lg = logf(fmaxf(g[(long long)(b0 + tid) * g_stride + h], 1e-38f));
      w = wgt ? wgt[(long long)(b0 + tid) * heads + h] : 1.f;
    }
#pragma unroll
    for (int o = 1; o < RC_LC; o <<= 1) {
      const float up = __shfl_up(lg, o, JV_WAVE);
      if (tid >= o) lg += up;
    }
    cl[tid] = lg;
    bs[tid] = w;
    gs[tid] = expf(lg);
    if (tid < n) cum[(long long)(b0 + tid) * heads + h] = expf(lg);
  }
  for (int i = tid; i < RC_LC * dq; i += 256) {
    const int j = i / dq, d = i - j * dq;
    float qv = 0.f, kv = 0.f;
    if (j < n && d < dim) {
      qv = q[(long long)(b0 + j) * ldq + hk * dim + d];
      kv = k[(long long)(b0 + j) * ldk + hk * dim + d];
    }
    qs[i] = qv;
    ks[i] = kv;
  }
  __syncthreads();
  {  // A (below the diagonal) and B (with the diagonal): thread (i, 4 consecutive j)
    const int i = tid >> 3, j0 = (tid & 7) * 4;
    float da[4] = {0.f, 0.f, 0.f, 0.f}, db[4] = {0.f, 0.f, 0.f, 0.f};
    if (j0 <= i) {
      for (int d = 0; d < dim; ++d) {
        const float kv = ks[i * dq + d], qv = qs[i * dq + d];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float kj = ks[(j0 + u) * dq + d];
          da[u] = fmaf(kv, kj, da[u]);
          db[u] = fmaf(qv, kj, db[u]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u;
      const float f = (j <= i && i < n) ? expf(cl[i] - cl[j]) : 0.f;
      ma[i * lm + j] = j < i ? da[u] * f : 0.f;
      mb[i * lm + j] = db[u] * f;
    }
  }
  __syncthreads();
  if (tid < RC_LC) {   // column tid of T: t_i = beta_i (e_i - sum_{j<i} A_ij t_j); a column depends on itself only
    const int c = tid;
    for (int i = 0; i < RC_LC; ++i) {
      float acc = i == c ? 1.f : 0.f;
      for (int j = c; j < i; ++j) acc = fmaf(-ma[i * lm + j], mt[j * lm + c], acc);
      mt[i * lm + c] = i < c ? 0.f : bs[i] * acc;
    }
  }
  // Kd from the plain keys, meanwhile
  float* wk_c = wk_out + ((long long)ch * heads + h) * RC_LC * dim;
  float* kd_c = kd_out + ((long long)ch * heads + h) * RC_LC * dim;
  for (int e = tid; e < RC_LC * dim; e += 256) {
    const int i = e / dim, d = e - i * dim;
    kd_c[e] = i < n ? ks[i * dq + d] * expf(cl[n - 1] - cl[i]) : 0.f;
  }
  __syncthreads();
  {  // B T into A's place; keys times G in place
    const int i = tid >> 3, j0 = (tid & 7) * 4;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int m = j0; m <= i; ++m) {
      const float b = mb[i * lm + m];
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = fmaf(b, mt[m * lm + j0 + u], acc[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) ma[i * lm + j0 + u] = acc[u];
    for (int e = tid; e < RC_LC * dq; e += 256) ks[e] *= gs[e / dq];
  }
  __syncthreads();
  // Wk = T (G K);  Qt = G Q - (B T)(G K)
  for (int e = tid; e < RC_LC * dim; e += 256) {
    const int i = e / dim, d = e - i * dim;
    float a = 0.f, b = 0.f;
    for (int j = 0; j <= i; ++j) {
      const float kv = ks[j * dq + d];
      a = fmaf(mt[i * lm + j], kv, a);
      b = fmaf(ma[i * lm + j], kv, b);
    }
    wk_c[e] = a;
    if (i < n) qt_out[((long long)(b0 + i) * heads + h) * dim + d] = gs[i] * qs[i * dq + d] - b;
  }
  // Wv = T V and the chunk's own outputs (B T) V, a slice of columns at a time
  float* wv_c = wv_out + ((long long)ch * heads + h) * RC_LC * vdim;
  for (int c0 = 0; c0 < vdim; c0 += RC_LV) {
    const int ncols = min(RC_LV, vdim - c0);
    __syncthreads();
    for (int i = tid; i < RC_LC * RC_LV; i += 256) {
      const int j = i / RC_LV, c = i % RC_LV;
      vs[i] = (j < n && c < ncols) ? v[(long long)(b0 + j) * ldv + h * vdim + c0 + c] : 0.f;
    }
    __syncthreads();
    for (int e = tid; e < RC_LC * (RC_LV / 4); e += 256) {
      const int i = e / (RC_LV / 4), c = (e % (RC_LV / 4)) * 4;
      if (c >= ncols) continue;
      float4 wv = {0.f, 0.f, 0.f, 0.f}, o = {0.f, 0.f, 0.f, 0.f};
      for (int j = 0; j <= i; ++j) {
        const float t = mt[i * lm + j], a = ma[i * lm + j];
        const float4 x = *(const float4*)(vs + j * RC_LV + c);
        wv.x = fmaf(t, x.x, wv.x); wv.y = fmaf(t, x.y, wv.y); wv.z = fmaf(t, x.z, wv.z); wv.w = fmaf(t, x.w, wv.w);
        o.x = fmaf(a, x.x, o.x); o.y = fmaf(a, x.y, o.y); o.z = fmaf(a, x.z, o.z); o.w = fmaf(a, x.w, o.w);
      }
      float* wd = wv_c + (long long)i * vdim + c0 + c;
      const float wvv[4] = {wv.x, wv.y, wv.z, wv.w}, ov[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c + u < ncols) {
          wd[u] = wvv[u];
          if (i < n) out[(long long)(b0 + i) * heads * vdim + h * vdim + c0 + c + u] = ov[u];
        }
    }
  }
}

#define RC_DS 32        // columns of the state a block of the delta scan keeps
// A barrier that waits for the block's LDS traffic only: loads from global memory that were asked for a turn ahead stay
// in flight across it (`__syncthreads` would wait for them too).
__device__ __forceinline__ void rc_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// grid (requests, heads, column slices of RC_DS).  Both products of a chunk run on the matrix cores in true 32-bit:
// U = Wv - Wk S with the key size shared out to the four waves (their shares are added through LDS), then
// S <- G S + Kd^T U with wave w owning rows 32 w .. 32 w + 31 of the slice in its accumulators for the whole walk.
__global__ void __launch_bounds__(256)
delta_scan_kernel(float* __restrict__ sb, float* __restrict__ state, const float* __restrict__ wk_in,
                  const float* __restrict__ kd_in, const float* __restrict__ wv_in, const float* __restrict__ cum,
                  const int* __restrict__ slot_ids, const int* __restrict__ req_chunks, const int* __restrict__ work,
                  const int* __restrict__ cu_seqlens, int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int r = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * RC_DS;
  const int first = req_chunks[r], last = req_chunks[r + 1];
  if (last <= first) return;
  const int dq = dim + 1, lu = RC_DS + 1;
  float* ss = lds;                       // [dim][RC_DS]: the slice of S, as the first product's operand
  float* wkd = ss + dim * RC_DS;         // [LC][dq]: Wk, then Kd
  float* us = wkd + RC_LC * dq;          // [LC][RC_DS + 1]: Wv, then U
  float* ps = us + RC_LC * lu;           // [4][LC][RC_DS + 1]: the waves' shares of Wk S
  const int tid = threadIdx.x;
  const int wave = tid / JV_WAVE, lane = tid % JV_WAVE, col = lane % 32, kh = lane / 32;
  const int ncols = min(RC_DS, vdim - c0);
  const bool live = col < ncols;
  float* S = state + ((long long)slot_ids[r] * heads + h) * dim * vdim + c0;
  for (int e = tid; e < dim * RC_DS; e += 256) {
    const int d = e / RC_DS, c = e % RC_DS;
    ss[e] = c < ncols ? S[(long long)d * vdim + c] : 0.f;
  }
  rc_f32x16 acc;                         // rows 32 wave + (e / 4) * 8 + kh * 4 + e % 4 of column col
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int d = wave * 32 + (e / 4) * 8 + kh * 4 + e % 4;
    acc[e] = (d < dim && live) ? S[(long long)d * vdim + col] : 0.f;
  }
  const int end = cu_seqlens[r + 1];
  // a chunk's Wk, Kd and Wv travel through registers: they are asked for a turn ahead, while the turn before computes
  constexpr int RK = RC_LC * 128 / 256, RU = RC_LC * RC_DS / 256;
  float rw[RK], rk[RK], ru[RU];
  int at[RK];            // where a thread's pieces of Wk and Kd go in LDS (-1: beyond the chunk)
#pragma unroll
  for (int u = 0; u < RK; ++u) {
    const int e = tid + u * 256;
    at[u] = e < RC_LC * dim ? (e / dim) * dq + e % dim : -1;
  }
  auto fetch_w = [&](int ch) {
    const float* wk_c = wk_in + ((long long)ch * heads + h) * RC_LC * dim;
    const float* wv_c = wv_in + ((long long)ch * heads + h) * RC_LC * vdim + c0;
#pragma unroll
    for (int u = 0; u < RK; ++u) rw[u] = wk_c[min(tid + u * 256, RC_LC * dim - 1)];   // beyond the chunk: its last element, unused
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int e = tid + u * 256, i = e / RC_DS, c = e % RC_DS;
      ru[u] = wv_c[(long long)i * vdim + min(c, ncols - 1)];
    }
  };
  auto fetch_k = [&](int ch) {
    const float* kd_c = kd_in + ((long long)ch * heads + h) * RC_LC * dim;
#pragma unroll
    for (int u = 0; u < RK; ++u) rk[u] = kd_c[min(tid + u * 256, RC_LC * dim - 1)];
  };
  fetch_w(first);
  fetch_k(first);
  const int share = dim / 4, d0 = wave * share;            // dim is a multiple of 4; a share may be odd
  for (int ch = first; ch < last; ++ch) {
    float* sb_c = sb + ((long long)ch * heads + h) * dim * vdim + c0;
    rc_lds_barrier();      // the turn before has written ss and read wkd and us
#pragma unroll
    for (int u = 0; u < RK; ++u)
      if (at[u] >= 0) wkd[at[u]] = rw[u];
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int e = tid + u * 256, i = e / RC_DS, c = e % RC_DS;
      us[i * lu + c] = c < ncols ? ru[u] : 0.f;
    }
    for (int e = tid; e < dim * RC_DS; e += 256) {       // the state before this chunk, for `apply`
      const int d = e / RC_DS, c = e % RC_DS;
      if (c < ncols) sb_c[(long long)d * vdim + c] = ss[e];
    }
    rc_lds_barrier();
    fetch_w(min(ch + 1, last - 1));     // never conditional: the last turn asks for its own chunk again
    {  // this wave's share of Wk S
      rc_f32x16 p = {};
      for (int d = 0; d < share; d += 2) {
        const int dd = d0 + d + kh;
        const bool in = d + kh < share;
        p = __builtin_amdgcn_mfma_f32_32x32x2f32(in ? wkd[col * dq + dd] : 0.f, in ? ss[dd * RC_DS + col] : 0.f, p, 0, 0, 0);
      }
      float* mine = ps + wave * RC_LC * lu;
#pragma unroll
      for (int e = 0; e < 16; ++e) mine[((e / 4) * 8 + kh * 4 + e % 4) * lu + col] = p[e];
    }
    rc_lds_barrier();
#pragma unroll
    for (int u = 0; u < RK; ++u)
      if (at[u] >= 0) wkd[at[u]] = rk[u];
#pragma unroll
    for (int u = 0; u < RU; ++u) {      // U = Wv - Wk S
      const int e = tid + u * 256, o = (e / RC_DS) * lu + e % RC_DS;
      us[o] -= (ps[o] + ps[RC_LC * lu + o]) + (ps[2 * RC_LC * lu + o] + ps[3 * RC_LC * lu + o]);
    }
    fetch_k(min(ch + 1, last - 1));
    rc_lds_barrier();
    const int b0 = work[2 * ch + 1];
    const int n = min(RC_LC, end - b0);
    const float gn = cum[(long long)(b0 + n - 1) * heads + h];
    if (wave * 32 < dim) {               // S = G S + Kd^T U: this wave's 32 rows
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] *= gn;
      const bool row_in = wave * 32 + col < dim;
      for (int j = 0; j < RC_LC; j += 2) {
        const int jj = j + kh;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(row_in ? wkd[jj * dq + wave * 32 + col] : 0.f, us[jj * lu + col], acc, 0, 0, 0);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int d = wave * 32 + (e / 4) * 8 + kh * 4 + e % 4;
        if (d < dim) ss[d * RC_DS + col] = acc[e];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int d = wave * 32 + (e / 4) * 8 + kh * 4 + e % 4;
    if (d < dim && live) S[(long long)d * vdim + col] = acc[e];
  }
}

// scratch: floats for chunks * heads * (2 * LC * dim + LC * vdim + dim * vdim) + tokens * heads * dim; cum: tokens * heads
extern "C" long long jv_delta_chunks_scratch_floats(int chunks, int tokens, int heads, int dim, int vdim) {
  return (long long)chunks * heads * (2LL * RC_LC * dim + (long long)RC_LC * vdim + (long long)dim * vdim) +
         (long long)tokens * heads * dim;
}

extern "C" int jv_delta_chunks(float* out, const float* q, long long ldq, const float* k, long long ldk,
                               const float* v, long long ldv, const float* g, int g_stride, const float* wgt,
                               float* state, const int* slot_ids, const int* cu_seqlens, int n_requests, int n_tokens,
                               int heads, int qk_heads, int dim, int vdim, int chunks, const int* work,
                               const int* req_chunks, float* scratch, float* cum, void* stream) {
  if (n_requests <= 0 || heads <= 0 || chunks <= 0) return 0;
  if (dim <= 0 || dim > 128 || dim % 4 || vdim <= 0 || heads > 65535 || qk_heads <= 0 || heads % qk_heads || !work ||
      !req_chunks || !scratch || !cum)
    return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  const long long per = (long long)chunks * heads;
  float* wk = scratch;
  float* kd = wk + per * RC_LC * dim;
  float* wv = kd + per * RC_LC * dim;
  float* sb = wv + per * RC_LC * vdim;
  float* qt = sb + per * dim * vdim;
  const size_t lds_local = (2 * RC_LC * (dim + RC_PAD) + 3 * RC_LC * (RC_LC + 1) + RC_LC * RC_LV + 3 * RC_LC) * sizeof(float);
  const size_t lds_scan = ((size_t)dim * RC_DS + RC_LC * (dim + 1) + 5 * RC_LC * (RC_DS + 1)) * sizeof(float);
  const size_t lds_apply = (size_t)RC_LC * (dim + 1) * sizeof(float);
  hipLaunchKernelGGL(delta_local_kernel, dim3(chunks, heads), dim3(256), lds_local, s, out, wk, kd, wv, qt, cum, q, ldq,
                     k, ldk, v, ldv, g, g_stride, wgt, work, cu_seqlens, heads, qk_heads, dim, vdim);
  hipLaunchKernelGGL(delta_scan_kernel, dim3(n_requests, heads, (vdim + RC_DS - 1) / RC_DS), dim3(256), lds_scan, s, sb,
                     state, wk, kd, wv, cum, slot_ids, req_chunks, work, cu_seqlens, heads, dim, vdim);
  hipLaunchKernelGGL(recurrence_apply_kernel, dim3(chunks, heads, (vdim + RC_LV - 1) / RC_LV), dim3(256), lds_apply, s,
                     out, sb, (const float*)nullptr, qt, (long long)heads * dim, work, cu_seqlens, heads, heads, dim, vdim);
  return JV_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- norm in groups with a gate
//   a = gate_first ? o * act(gate) : o;   y = a * rsqrt(mean_group(a^2) + eps) * w[c % w_period];
//   out = T( (gate_first ? y : y * act(gate)) * out_scale );   act: 1 silu, 2 sigmoid;  w null: no weight
// grid (rows, ceil(groups / 4)); one wave a group.
template <typename T>
__global__ void __launch_bounds__(256)
group_gated_norm_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate,
                        long long g_stride, const float* __restrict__ w, int w_period, int width, int group,
                        float eps, int gate_act, int gate_first, float out_scale) {
  const long long t = blockIdx.x;
  const int grp = blockIdx.y * 4 + threadIdx.x / JV_WAVE, lane = threadIdx.x % JV_WAVE;
  if (grp * group >= width) return;
  const float* x = o + t * width + grp * group;
  const T* gp = gate + t * g_stride + grp * group;
  float ss = 0.f;
  for (int i = lane; i < group; i += JV_WAVE) {
    float a = x[i];
    if (gate_first) {
      const float z = to_f32(gp[i]);
      a *= gate_act == 1 ? rc_silu(z) : 1.f / (1.f + expf(-z));
    }
    ss = fmaf(a, a, ss);
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)group + eps) * out_scale;
  for (int i = lane; i < group; i += JV_WAVE) {
    const float z = to_f32(gp[i]);
    const float ga = gate_act == 1 ? rc_silu(z) : 1.f / (1.f + expf(-z));
    const float wv = w ? w[(grp * group + i) % w_period] : 1.f;
    out[t * width + grp * group + i] = from_f32<T>(x[i] * ga * inv * wv);
  }
}

// The same for wide groups: one block a (row, group).
template <typename T>
__global__ void __launch_bounds__(1024)
group_gated_norm_block_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate,
                              long long g_stride, const float* __restrict__ w, int w_period, int width, int group,
                              float eps, int gate_act, int gate_first, float out_scale) {
  __shared__ float red[32];
  const long long t = blockIdx.x;
  const int grp = blockIdx.y;
  const float* x = o + t * width + grp * group;
  const T* gp = gate + t * g_stride + grp * group;
  float ss = 0.f;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    float a = x[i];
    if (gate_first) {
      const float z = to_f32(gp[i]);
      a *= gate_act == 1 ? rc_silu(z) : 1.f / (1.f + expf(-z));
    }
    ss = fmaf(a, a, ss);
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)group + eps) * out_scale;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    const float z = to_f32(gp[i]);
    const float ga = gate_act == 1 ? rc_silu(z) : 1.f / (1.f + expf(-z));
    const float wv = w ? w[(grp * group + i) % w_period] : 1.f;
    out[t * width + grp * group + i] = from_f32<T>(x[i] * ga * inv * wv);
  }
}

extern "C" int jv_recurrence_max_dim() { return RC_ROWS * 256; }
extern "C" int jv_short_conv_max_taps() { return RC_MAX_LAGS + 1; }

extern "C" int jv_head_unit_norm(float* x, long long ld, long long n, int heads, int d, float eps, int heads_a,
                                 float scale_a, float scale_b, void* stream) {
  if (n <= 0 || heads <= 0 || d <= 0) return 0;
  if ((long long)heads * d > ld) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(head_unit_norm_kernel, dim3((unsigned)((n * heads + 3) / 4)), dim3(256), 0, (hipStream_t)stream, x,
                     ld, n, heads, d, eps, heads_a, scale_a, scale_b);
  return JV_LAUNCH_CHECK();
}

extern "C" int jv_recurrence_steps(float* out, const float* q, long long ldq, const float* k, long long ldk,
                                   const float* v, long long ldv, const float* g, int g_stride, const float* wgt,
                                   const float* skip, float* state, const int* slot_ids, const int* cu_seqlens,
                                   int n_requests, int heads, int qk_heads, int dim, int vdim, int delta,
                                   void* stream) {
  if (n_requests <= 0 || heads <= 0) return 0;
  if (dim <= 0 || vdim <= 0 || heads > 65535 || qk_heads <= 0 || heads % qk_heads) return (int)hipErrorInvalidValue;
  int cols = 64;                       /* the widest slice that keeps a thread's rows in registers */
  while (cols > 1 && (cols / 2 >= vdim || (long long)dim * cols > 256LL * RC_ROWS)) cols /= 2;
  if ((long long)dim * cols > 256LL * RC_ROWS) return (int)hipErrorInvalidValue;
  const int parts = 256 / cols;
  const size_t shmem = (2 * (2 * dim + cols) + 2 * parts * cols) * sizeof(float);
  hipLaunchKernelGGL(recurrence_steps_kernel, dim3(n_requests, heads, (vdim + cols - 1) / cols), dim3(256), shmem,
                     (hipStream_t)stream, out, q, ldq, k, ldk, v, ldv, g, g_stride, wgt, skip, state, slot_ids,
                     cu_seqlens, heads, qk_heads, dim, vdim, cols, delta);
  return JV_LAUNCH_CHECK();
}

#define DEFINE_RECURRENCE(SUF, T)                                                                              \
  extern "C" int jv_short_conv_##SUF(float* out, long long ldo, const void* proj, long long ld, int c_off,     \
                                     int channels, int taps, const float* w, const float* bias, float* state,  \
                                     const int* slot_ids, const int* cu_seqlens, int n_requests,               \
                                     int max_q_len, int act, void* stream) {                                   \
    if (n_requests <= 0 || channels <= 0 || max_q_len <= 0) return 0;                                          \
    if (taps < 1 || taps > RC_MAX_LAGS + 1) return (int)hipErrorInvalidValue;                                  \
    const int seg_len = 64;                                                                                    \
    hipLaunchKernelGGL(short_conv_kernel<T>, dim3(n_requests, (channels + 255) / 256,                          \
                                                  (max_q_len + seg_len - 1) / seg_len),                        \
                       dim3(256), 0, (hipStream_t)stream, out, ldo, (const T*)proj, ld, c_off, channels, taps, \
                       w, bias, state, slot_ids, cu_seqlens, act, seg_len);                                    \
    return JV_LAUNCH_CHECK();                                                                                  \
  }                                                                                                            \
  extern "C" int jv_recurrence_gates_##SUF(float* g, float* wgt, const void* proj, long long ld, int dt_off,   \
                                           int w_off, const float* dt_bias, const float* a_log, int n,         \
                                           int heads, int mode, void* stream) {                                \
    if (n <= 0 || heads <= 0) return 0;                                                                        \
    hipLaunchKernelGGL(recurrence_gates_kernel<T>, dim3((unsigned)(((long long)n * heads + 255) / 256)),       \
                       dim3(256), 0, (hipStream_t)stream, g, wgt, (const T*)proj, ld, dt_off, w_off, dt_bias,  \
                       a_log, n, heads, mode);                                                                 \
    return JV_LAUNCH_CHECK();                                                                                  \
  }                                                                                                            \
  extern "C" int jv_heads_to_f32_##SUF(float* out, const void* proj, long long ld, int off, int n, int heads,  \
                                       int d, int rot_dims, const float* cos_sin, float scale, void* stream) { \
    if (n <= 0 || heads <= 0 || d <= 0) return 0;                                                              \
    if (rot_dims < 0 || rot_dims > d || rot_dims % 2 || (rot_dims && !cos_sin)) return (int)hipErrorInvalidValue; \
    hipLaunchKernelGGL(heads_to_f32_kernel<T>, dim3((unsigned)(((long long)n * heads * d + 255) / 256)),       \
                       dim3(256), 0, (hipStream_t)stream, out, (const T*)proj, ld, off, n, heads, d, rot_dims, \
                       cos_sin, scale);                                                                        \
    return JV_LAUNCH_CHECK();                                                                                  \
  }                                                                                                            \
  extern "C" int jv_qkv_to_f32_##SUF(float* out, const void* proj, long long ld, int n, int heads, int d,      \
                                     int dv, int rot_dims, const float* cos_sin, float k_scale, void* stream) { \
    if (n <= 0 || heads <= 0 || d <= 0 || dv <= 0) return 0;                                                   \
    if (rot_dims < 0 || rot_dims > d || rot_dims % 2 || (rot_dims && !cos_sin)) return (int)hipErrorInvalidValue; \
    const long long total = (long long)n * (2LL * heads * d + (long long)heads * dv);                          \
    hipLaunchKernelGGL(qkv_to_f32_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,              \
                       (hipStream_t)stream, out, (const T*)proj, ld, n, heads, d, dv, rot_dims, cos_sin,       \
                       k_scale);                                                                               \
    return JV_LAUNCH_CHECK();                                                                                  \
  }                                                                                                            \
  extern "C" int jv_group_gated_norm_##SUF(void* out, const float* o, const void* gate, long long g_stride,    \
                                           const float* w, int w_period, int n, int width, int group,          \
                                           float eps, int gate_act, int gate_first, float out_scale,           \
                                           void* stream) {                                                     \
    if (n <= 0 || width <= 0) return 0;                                                                        \
    if (group <= 0 || width % group || (w && w_period <= 0) || (gate_act != 1 && gate_act != 2))               \
      return (int)hipErrorInvalidValue;                                                                        \
    const int groups = width / group;                                                                          \
    if (groups > 65535) return (int)hipErrorInvalidValue;                                                      \
    if (group >= 256) {                                                                                        \
      /* few rows of very wide groups (a decode step): more threads a row, the row's time is its chain of loads */ \
      const int threads = (group >= 2048 && (long long)n * groups <= 256) ? 1024 : 256;                       \
      hipLaunchKernelGGL(group_gated_norm_block_kernel<T>, dim3(n, groups), dim3(threads), 0, (hipStream_t)stream, \
                         (T*)out, o, (const T*)gate, g_stride, w, w_period, width, group, eps, gate_act,       \
                         gate_first, out_scale);                                                               \
      return JV_LAUNCH_CHECK();                                                                                \
    }                                                                                                          \
    hipLaunchKernelGGL(group_gated_norm_kernel<T>, dim3(n, (groups + 3) / 4), dim3(256), 0,                    \
                       (hipStream_t)stream, (T*)out, o, (const T*)gate, g_stride, w, w_period, width, group,   \
                       eps, gate_act, gate_first, out_scale);                                                  \
    return JV_LAUNCH_CHECK();                                                                                  \
  }

DEFINE_RECURRENCE(bf16, bf16_t)
DEFINE_RECURRENCE(f32, float)
