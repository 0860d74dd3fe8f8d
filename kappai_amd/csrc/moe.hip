// Mixture of experts: router, the step's rows sorted by expert, the experts' products over that
// order, and the weighted sum.  Nothing is read back by the host: every launch is sized by the
// number of rows alone, so a step with experts can be captured in a graph.
//   moe_route     z = W_router h in float32, the `top` largest chosen (lowest index on ties),
//                 weights = softmax over the chosen logits
//   moe_plan      (row, choice) pairs in expert order, every expert's run starting on a tile of
//                 MOE_TILE_M slots: slot_of_pair, pair_of_slot (-1: empty), tile_expert (-1: unused)
//   moe_gemm      tile by tile: act = silu(x Wg^T) * (x Wu^T) on gathered rows, or y = act Wd^T
//   moe_combine   out[t] = sum_k weight[t, k] * y[slot of (t, k)], in the order of k, float32
#include "common.h"

#define MOE_TILE_M 32
#define MOE_TILE_N 64
#define MOE_TILE_K 32
#define MOE_MAX_TOP 16
#define MOE_THREADS 256

extern "C" int kappai_moe_tile_rows() { return MOE_TILE_M; }

template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_route_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ router, int n_rows, int D, int E,
    int top, int* __restrict__ idx, float* __restrict__ wts) {
  extern __shared__ float logits_all[];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int row_raw = blockIdx.x * (MOE_THREADS / WAVE) + wave;
  const int row = row_raw < n_rows ? row_raw : n_rows - 1;
  float* logits = logits_all + wave * E;
  const T* xr = x + (size_t)row * ldx;
  for (int e = 0; e < E; ++e) {
    const float* r = router + (size_t)e * D;
    float acc = 0.f;
    for (int c = lane; c < D; c += WAVE) acc = fmaf(to_f32(xr[c]), r[c], acc);
    acc = wave_sum(acc);
    if (lane == 0) logits[e] = acc;
  }
  __syncthreads();
  float cv[MOE_MAX_TOP];
  int ci[MOE_MAX_TOP];
#pragma unroll
  for (int k = 0; k < MOE_MAX_TOP; ++k) {
    if (k < top) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int e = lane; e < E; e += WAVE) {
        const float v = logits[e];
        if (v > best) { best = v; at = e; }      // the lowest index among a lane's equals
      }
      const float m = wave_max(best);
      const int who = -wave_max(best == m ? -at : -0x7fffffff);
      cv[k] = m;
      ci[k] = who;
      __syncthreads();
      if (lane == 0 && who < E) logits[who] = -INFINITY;
      __syncthreads();
    }
  }
  if (lane == 0 && row_raw < n_rows) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < MOE_MAX_TOP; ++k)
      if (k < top) sum += expf(cv[k] - cv[0]);
#pragma unroll
    for (int k = 0; k < MOE_MAX_TOP; ++k)
      if (k < top) {
        idx[(size_t)row * top + k] = ci[k] < E ? ci[k] : 0;
        wts[(size_t)row * top + k] = expf(cv[k] - cv[0]) / sum;
      }
  }
}

extern "C" int kappai_moe_route(const void* x, int ldx, int x_is_bf16, const float* router, int T,
                                int D, int E, int top, int* idx, float* wts, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || top > MOE_MAX_TOP || top > E || E > 4096) return (int)hipErrorInvalidValue;
  const int waves = MOE_THREADS / WAVE;
  const dim3 grid((T + waves - 1) / waves);
  const size_t lds = (size_t)waves * E * sizeof(float);
  if (x_is_bf16)
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, dim3(MOE_THREADS), lds, stream,
                       (const bf16_t*)x, ldx, router, T, D, E, top, idx, wts);
  else
    hipLaunchKernelGGL(moe_route_kernel<float>, grid, dim3(MOE_THREADS), lds, stream,
                       (const float*)x, ldx, router, T, D, E, top, idx, wts);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// One wave sorts the pairs by expert, stably: 64 pairs at a time, the lanes with the same expert
// found by ballots, their places by counting the lanes below.  Pass 1 counts, pass 2 places.
__global__ __launch_bounds__(WAVE) void moe_plan_kernel(
    const int* __restrict__ idx, int P, int E, int n_tiles, int* __restrict__ slot_of_pair,
    int* __restrict__ pair_of_slot, int* __restrict__ tile_expert) {
  extern __shared__ int plan_lds[];
  int* count = plan_lds;           // pairs of the expert; in pass 2: pairs placed so far
  int* base = plan_lds + E;        // first slot of the expert
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += WAVE) count[e] = 0;
  for (int i = lane; i < n_tiles * MOE_TILE_M; i += WAVE) pair_of_slot[i] = -1;
  for (int i = lane; i < n_tiles; i += WAVE) tile_expert[i] = -1;
  __syncthreads();
  for (int pass = 0; pass < 2; ++pass) {
    for (int p0 = 0; p0 < P; p0 += WAVE) {
      const int p = p0 + lane;
      const int e = p < P ? idx[p] : -1;
      bool todo = p < P;
      while (true) {
        const unsigned long long rest = __ballot(todo);
        if (!rest) break;
        const int leader = __ffsll((long long)rest) - 1;
        const int cur = __shfl(e, leader);
        const bool mine = todo && e == cur;
        const unsigned long long mask = __ballot(mine);
        const int before = count[cur];
        __syncthreads();
        if (pass == 1 && mine) {
          const int rank = __popcll(mask & ((1ull << lane) - 1ull));
          const int slot = base[cur] + before + rank;
          slot_of_pair[p] = slot;
          pair_of_slot[slot] = p;
        }
        if (lane == 0) count[cur] = before + __popcll(mask);
        __syncthreads();
        if (mine) todo = false;
      }
    }
    if (pass == 0) {
      if (lane == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
          base[e] = at;
          const int tiles = (count[e] + MOE_TILE_M - 1) / MOE_TILE_M;
          for (int i = 0; i < tiles; ++i) tile_expert[at / MOE_TILE_M + i] = e;
          at += tiles * MOE_TILE_M;
          count[e] = 0;
        }
      }
      __syncthreads();
    }
  }
}

extern "C" int kappai_moe_plan(const int* idx, int P, int E, int n_tiles, int* slot_of_pair,
                               int* pair_of_slot, int* tile_expert, hipStream_t stream) {
  if (P <= 0) return 0;
  if (E < 1 || E > 4096 || n_tiles < P / MOE_TILE_M + (E < P ? E : P))
    return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(WAVE), 2 * (size_t)E * sizeof(int), stream,
                     idx, P, E, n_tiles, slot_of_pair, pair_of_slot, tile_expert);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

__device__ __forceinline__ float silu_exact(float g) { return g / (1.0f + expf(-g)); }

// A tile of MOE_TILE_M slots of one expert times MOE_TILE_N rows of its matrix, float sums on
// the vector units (this is the 32-bit path, and the path of any shape).  GATED: the rows are
// gathered from x by pair / top, two matrices, out = silu(g) * u in T; else the rows are the
// slots of `a` themselves and out is float.
template <typename T, int GATED>
__global__ __launch_bounds__(MOE_THREADS) void moe_gemm_kernel(
    const T* __restrict__ a, int lda, const T* __restrict__ w0, const T* __restrict__ w1, int N,
    int K, const int* __restrict__ tile_expert, const int* __restrict__ pair_of_slot, int top,
    void* __restrict__ out_v) {
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  __shared__ float As[MOE_TILE_K][MOE_TILE_M + 1];
  __shared__ float W0s[MOE_TILE_K][MOE_TILE_N + 1];
  __shared__ float W1s[GATED ? MOE_TILE_K : 1][MOE_TILE_N + 1];
  __shared__ int src_row[MOE_TILE_M];
  const int tid = threadIdx.x;
  if (tid < MOE_TILE_M) {
    const int slot = tile * MOE_TILE_M + tid;
    const int pair = pair_of_slot[slot];
    src_row[tid] = pair < 0 ? -1 : (GATED ? pair / top : slot);
  }
  __syncthreads();
  const int n0 = blockIdx.y * MOE_TILE_N;
  const T* W0 = w0 + (size_t)e * N * K;
  const T* W1 = GATED ? w1 + (size_t)e * N * K : nullptr;
  const int ty = tid / 16, tx = tid % 16;
  float acc0[2][4] = {}, acc1[2][4] = {};
  const int am = tid / 8, ak = (tid % 8) * 4;       // this thread's piece of the A tile
  const int wn = tid / 4, wk = (tid % 4) * 8;       // and of the W tiles
  for (int k0 = 0; k0 < K; k0 += MOE_TILE_K) {
    const int r = src_row[am];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + ak + i;
      As[ak + i][am] = (r >= 0 && k < K) ? to_f32(a[(size_t)r * lda + k]) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + wk + i, n = n0 + wn;
      const bool ok = n < N && k < K;
      W0s[wk + i][wn] = ok ? to_f32(W0[(size_t)n * K + k]) : 0.f;
      if (GATED) W1s[wk + i][wn] = ok ? to_f32(W1[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < MOE_TILE_K; ++k) {
      const float a0 = As[k][2 * ty], a1 = As[k][2 * ty + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b0 = W0s[k][tx + 16 * j];
        acc0[0][j] = fmaf(a0, b0, acc0[0][j]);
        acc0[1][j] = fmaf(a1, b0, acc0[1][j]);
        if (GATED) {
          const float b1 = W1s[k][tx + 16 * j];
          acc1[0][j] = fmaf(a0, b1, acc1[0][j]);
          acc1[1][j] = fmaf(a1, b1, acc1[1][j]);
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = 2 * ty + i;
    if (src_row[m] < 0) continue;
    const size_t slot = (size_t)tile * MOE_TILE_M + m;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      if (GATED)
        from_f32((T*)out_v + slot * N + n, silu_exact(acc0[i][j]) * acc1[i][j]);
      else
        ((float*)out_v)[slot * N + n] = acc0[i][j];
    }
  }
}

extern "C" int kappai_moe_gemm(const void* a, int lda, const void* w0, const void* w1, int N,
                               int K, const int* tile_expert, const int* pair_of_slot, int top,
                               int n_tiles, void* out, int gated, int is_bf16,
                               hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  const dim3 grid(n_tiles, (N + MOE_TILE_N - 1) / MOE_TILE_N);
  if (grid.y > 65535) return (int)hipErrorInvalidValue;
#define MOE_GEMM_LAUNCH(TT, G)                                                                  \
  hipLaunchKernelGGL((moe_gemm_kernel<TT, G>), grid, dim3(MOE_THREADS), 0, stream, (const TT*)a, \
                     lda, (const TT*)w0, (const TT*)w1, N, K, tile_expert, pair_of_slot, top, out)
  if (is_bf16) {
    if (gated) MOE_GEMM_LAUNCH(bf16_t, 1); else MOE_GEMM_LAUNCH(bf16_t, 0);
  } else {
    if (gated) MOE_GEMM_LAUNCH(float, 1); else MOE_GEMM_LAUNCH(float, 0);
  }
#undef MOE_GEMM_LAUNCH
  KAPPAI_RETURN_LAUNCH_STATUS();
}

__global__ __launch_bounds__(MOE_THREADS) void moe_combine_kernel(
    const float* __restrict__ y, const int* __restrict__ slot_of_pair,
    const float* __restrict__ wts, int top, int D, float* __restrict__ out) {
  const int t = blockIdx.x;
  for (int n = threadIdx.x; n < D; n += MOE_THREADS) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc = fmaf(wts[(size_t)t * top + k], y[(size_t)slot_of_pair[(size_t)t * top + k] * D + n],
                 acc);
    out[(size_t)t * D + n] = acc;
  }
}

extern "C" int kappai_moe_combine(const float* y, const int* slot_of_pair, const float* wts, int T,
                                  int top, int D, float* out, hipStream_t stream) {
  if (T <= 0) return 0;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(MOE_THREADS), 0, stream, y, slot_of_pair,
                     wts, top, D, out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
