// The two grouped products of routed experts on the matrix cores (bfloat16, float accumulation); the
// grouping they read (tiles of 64 or 128 rows of one expert each) is made by moe.hip.
//
// A block of 4 waves takes one tile of (token, choice) rows against 64 rows of the expert's weight and
// walks the inner size in chunks of 64: the rows of x (gathered by token) and of W go through LDS, the
// next chunk's global loads are asked for (unconditionally, clamped) before the current chunk is
// multiplied.  v_mfma_f32_16x16x32_bf16 with A = 16 rows of W (wave w owns rows 16 w .. 16 w + 15 of the
// tile), B = 16 rows of x: the accumulator of row tile mt holds y^T[n = 4 lc + e][m = 16 mt + li].
// Each output row is a sum over the inner size in a fixed order, whatever else is in the step.
//   GATED:  z[pos] = act(w g) * (w u), g = Wg[e] x[token], u = Wu[e] x[token]       (bf16)
//   else:   y[kk][token] = (Wd[e] z[pos]) * w_out                                   (float)
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define MM_T 64            // rows of a tile, rows of W of a block, columns of a chunk
#define MM_S 80            // LDS row length: 40 dwords, 8 mod 16: 16-byte reads of 16 rows are conflict-free

// MT: row tiles of 16 a block takes (a tile of the grouping has 16 MT rows).  Without a grouping
// (tile_expert null) the product is a plain one: rows in order, one weight matrix, float output [rows, N].
template <bool GATED, int MT>
__global__ void __launch_bounds__(256)
moe_mfma_kernel(void* __restrict__ out, const bf16_t* __restrict__ a_rows, const bf16_t* __restrict__ W0,
                const bf16_t* __restrict__ W1, const int* __restrict__ meta, const int* __restrict__ offsets,
                const int* __restrict__ tile_expert, const int* __restrict__ tile_row0, const int* __restrict__ order,
                const float* __restrict__ weights, int top, int n_tokens, int K, int N, int act, int use_weight) {
  constexpr int TM = 16 * MT;
  if (tile_expert && (int)blockIdx.x >= meta[0]) return;
  __shared__ __attribute__((aligned(16))) bf16_t xs[TM * MM_S];
  __shared__ __attribute__((aligned(16))) bf16_t w0s[MM_T * MM_S];
  __shared__ __attribute__((aligned(16))) bf16_t w1s[GATED ? MM_T * MM_S : 8];
  __shared__ int ent[TM];
  const int e = tile_expert ? tile_expert[blockIdx.x] : 0, row0 = tile_expert ? tile_row0[blockIdx.x] : blockIdx.x * TM;
  const int rows = min(TM, (tile_expert ? offsets[e + 1] : n_tokens) - row0);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 15, lc = lane >> 4;
  const int n0 = blockIdx.y * MM_T;
  if (tid < TM) ent[tid] = tile_expert ? order[row0 + min(tid, rows - 1)] : row0 + min(tid, rows - 1);   // rows beyond the tile repeat its last row
  __syncthreads();
  // staging: thread t brings pieces t and t + 256 of each operand: piece p = row p / 8, columns (p % 8) * 8 .. + 7
  const int pr = tid >> 3, pc = (tid & 7) * 8;
  constexpr int XQ = TM / 32;        // pieces of x a thread brings
  const bf16_t* xrow[XQ];
  const bf16_t* w0row[2];
  const bf16_t* w1row[2];
#pragma unroll
  for (int q = 0; q < XQ; ++q) {
    const int r = pr + 32 * q;
    const long long src = GATED ? (long long)(ent[r] / top) : (long long)(row0 + min(r, rows - 1));
    xrow[q] = a_rows + src * K;
  }
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const long long wr = (long long)e * N + min(n0 + pr + 32 * q, N - 1);
    w0row[q] = W0 + wr * K;
    w1row[q] = GATED ? W1 + wr * K : W0;
  }
  bf16x8 rx[XQ], rw0[2], rw1[2];
  auto fetch = [&](int k0) {
    const int k = min(k0 + pc, K - 8);
#pragma unroll
    for (int q = 0; q < XQ; ++q) rx[q] = *(const bf16x8*)(xrow[q] + k);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      rw0[q] = *(const bf16x8*)(w0row[q] + k);
      if (GATED) rw1[q] = *(const bf16x8*)(w1row[q] + k);
    }
  };
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  f32x4 acc0[MT], acc1[GATED ? MT : 1];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc0[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (GATED) acc1[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += MM_T) {
    const bool inside = k0 + pc < K;          // a chunk's columns beyond the inner size are zeros of x
    __syncthreads();                          // the chunk before is multiplied
#pragma unroll
    for (int q = 0; q < XQ; ++q) *(bf16x8*)(xs + (pr + 32 * q) * MM_S + pc) = inside ? rx[q] : zero;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int at = (pr + 32 * q) * MM_S + pc;
      *(bf16x8*)(w0s + at) = rw0[q];
      if (GATED) *(bf16x8*)(w1s + at) = rw1[q];
    }
    __syncthreads();
    fetch(k0 + MM_T);                         // beyond the end: the last pieces again, never used
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int col = ks * 32 + lc * 8;
      const bf16x8 a0 = *(const bf16x8*)(w0s + (wave * 16 + li) * MM_S + col);
      bf16x8 a1 = zero;
      if (GATED) a1 = *(const bf16x8*)(w1s + (wave * 16 + li) * MM_S + col);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 b = *(const bf16x8*)(xs + (mt * 16 + li) * MM_S + col);
        acc0[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b, acc0[mt], 0, 0, 0);
        if (GATED) acc1[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b, acc1[mt], 0, 0, 0);
      }
    }
  }
  const int nb = n0 + wave * 16 + lc * 4;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + li;
    if (m >= rows) continue;
    const int s = ent[m];
    const float w = use_weight ? weights[s] : 1.f;
    if (GATED) {
      bf16_t* z = (bf16_t*)out + (long long)(row0 + m) * N;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (nb + c < N) z[nb + c] = from_f32<bf16_t>(jv_gated(act, acc0[mt][c] * w, acc1[mt][c] * w));
    } else {
      const int token = s / top, kk = s - token * top;
      float* y = (float*)out + ((long long)kk * n_tokens + token) * N;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (nb + c < N) y[nb + c] = acc0[mt][c] * w;
    }
  }
}

template <bool GATED>
static int launch_moe_mfma(int tile_rows, dim3 grid, hipStream_t stream, void* out, const bf16_t* a, const bf16_t* W0,
                           const bf16_t* W1, const int* meta, const int* offsets, const int* tile_expert,
                           const int* tile_row0, const int* order, const float* weights, int top, int n_tokens, int K,
                           int N, int act, int use_weight) {
  if (tile_rows == 128)
    hipLaunchKernelGGL((moe_mfma_kernel<GATED, 8>), grid, dim3(256), 0, stream, out, a, W0, W1, meta, offsets, tile_expert,
                       tile_row0, order, weights, top, n_tokens, K, N, act, use_weight);
  else if (tile_rows == 64)
    hipLaunchKernelGGL((moe_mfma_kernel<GATED, 4>), grid, dim3(256), 0, stream, out, a, W0, W1, meta, offsets, tile_expert,
                       tile_row0, order, weights, top, n_tokens, K, N, act, use_weight);
  else
    return (int)hipErrorInvalidValue;
  return JV_LAUNCH_CHECK();
}

// gate/up: x [tokens, hidden], Wg, Wu [experts, ff, hidden] -> z [entries, ff] bf16 by position; tile_rows (64 or
// 128) is what the grouping was made with
extern "C" int jv_moe_gate_up_mfma_bf16(void* z, const void* x, const void* Wg, const void* Wu, const int* meta,
                                        const int* offsets, const int* tile_expert, const int* tile_row0,
                                        const int* order, const float* weights, int max_tiles, int top, int hidden,
                                        int ff, int act, int scale_input, int tile_rows, void* stream) {
  if (max_tiles <= 0 || ff <= 0) return 0;
  if (!jv_act_known(act) || hidden < 8 || hidden % 8 || (ff + MM_T - 1) / MM_T > 65535) return (int)hipErrorInvalidValue;
  return launch_moe_mfma<true>(tile_rows, dim3(max_tiles, (ff + MM_T - 1) / MM_T), (hipStream_t)stream, z, (const bf16_t*)x,
                               (const bf16_t*)Wg, (const bf16_t*)Wu, meta, offsets, tile_expert, tile_row0, order,
                               weights, top, 0, hidden, ff, act, scale_input);
}

// down: z [entries, ff] by position, Wd [experts, hidden, ff] -> y [top, tokens, hidden] float
extern "C" int jv_moe_down_mfma_bf16(float* y, const void* z, const void* Wd, const int* meta, const int* offsets,
                                     const int* tile_expert, const int* tile_row0, const int* order,
                                     const float* weights, int max_tiles, int top, int n_tokens, int hidden, int ff,
                                     int scale_output, int tile_rows, void* stream) {
  if (max_tiles <= 0 || hidden <= 0) return 0;
  if (ff < 8 || ff % 8 || (hidden + MM_T - 1) / MM_T > 65535) return (int)hipErrorInvalidValue;
  return launch_moe_mfma<false>(tile_rows, dim3(max_tiles, (hidden + MM_T - 1) / MM_T), (hipStream_t)stream, y,
                                (const bf16_t*)z, (const bf16_t*)Wd, nullptr, meta, offsets, tile_expert, tile_row0, order,
                                weights, top, n_tokens, ff, hidden, 0, scale_output);
}

// y [M, N] float = x [M, K] W[N, K]^T for bfloat16 x and W: the same kernel without a grouping (router logits
// of many tokens).  K a multiple of 8.
extern "C" int jv_gemm_rows_f32out_bf16(float* y, const void* x, const void* W, int M, int N, int K, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K < 8 || K % 8 || (N + MM_T - 1) / MM_T > 65535) return (int)hipErrorInvalidValue;
  return launch_moe_mfma<false>(128, dim3((M + 127) / 128, (N + MM_T - 1) / MM_T), (hipStream_t)stream, y, (const bf16_t*)x,
                                (const bf16_t*)W, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 1, M, K, N, 0, 0);
}
