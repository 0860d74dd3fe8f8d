// Differential attention around the paged attention kernels.  A head has two score maps over the
// same values; each map is run as a head of its own by the framework's attention kernels, which
// want one head size D for queries, keys and values: the maps' queries and keys (size d) and the
// values (size dv) are widened with zeros to D, and a kv head's values are stored once per map.
//   map (h, m) of query head h = g R + i (R query heads a kv head) is attention head (2 g + m) R + i
//   and reads kv head 2 g + m, so that the kernels' rule "head / R" finds it.
// diff_store writes the widened queries and stores keys and values; diff_combine makes
// o = a1 - lambda a2, divides every head's o by its root mean square and scales it.
#include "common.h"

#define DA_THREADS 256

// proj [T, ld] = (q: H x 2 x d | k: G x 2 x d | v: G x dv), the two maps of a head side by side.
template <typename T>
__global__ __launch_bounds__(DA_THREADS) void diff_store_kernel(
    const T* __restrict__ proj, int ld, T* __restrict__ q_out, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int d, int dv, int D,
    int ps, int store_kv) {
  const int t = blockIdx.x;
  const T* p = proj + (size_t)t * ld;
  const int R = H / G;
  const T zero = T(0);
  // queries
  T* q = q_out + (size_t)t * 2 * H * D;
  for (int i = threadIdx.x; i < 2 * H * D; i += DA_THREADS) {
    const int c = i % D, head = i / D;          // head = (2 g + m) R + hi
    const int hi = head % R, gm = head / R, m = gm & 1, g = gm >> 1;
    q[i] = c < d ? p[((size_t)(g * R + hi) * 2 + m) * d + c] : zero;
  }
  if (!store_kv) return;
  const int pos = row_pos[t];
  const int page = block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  const int slot = pos % ps;
  const T* k = p + (size_t)H * 2 * d;
  const T* v = k + (size_t)G * 2 * d;
  T* kp = k_pool + (size_t)page * 2 * G * ps * D;
  T* vp = v_pool + (size_t)page * 2 * G * D * ps;
  for (int i = threadIdx.x; i < 2 * G * D; i += DA_THREADS) {
    const int c = i % D, gm = i / D, g = gm >> 1;
    kp[((size_t)gm * ps + slot) * D + c] = c < d ? k[(size_t)gm * d + c] : zero;
    vp[((size_t)gm * D + c) * ps + slot] = c < dv ? v[(size_t)g * dv + c] : zero;
  }
}

extern "C" int kappai_diff_store(const void* proj, int ld, void* q_out, void* k_pool, void* v_pool,
                                 const int* row_pos, const int* row_seg, const int* block_tables,
                                 int max_blocks, int T, int H, int G, int d, int dv, int D, int ps,
                                 int store_kv, int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H % G || d > D || dv > D) return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(diff_store_kernel<bf16_t>, dim3(T), dim3(DA_THREADS), 0, stream,
                       (const bf16_t*)proj, ld, (bf16_t*)q_out, (bf16_t*)k_pool, (bf16_t*)v_pool,
                       row_pos, row_seg, block_tables, max_blocks, H, G, d, dv, D, ps, store_kv);
  else
    hipLaunchKernelGGL(diff_store_kernel<float>, dim3(T), dim3(DA_THREADS), 0, stream,
                       (const float*)proj, ld, (float*)q_out, (float*)k_pool, (float*)v_pool,
                       row_pos, row_seg, block_tables, max_blocks, H, G, d, dv, D, ps, store_kv);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ctx [T, 2H, D] (the maps' outputs, in the order above) -> out [T, H, dv]: a wave a (row, head).
template <typename T>
__global__ __launch_bounds__(WAVE) void diff_combine_kernel(
    const T* __restrict__ ctx, T* __restrict__ out, int H, int G, int dv, int D, float lambda,
    float eps, float gain) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int R = H / G, g = h / R, hi = h % R;
  const T* a1 = ctx + ((size_t)t * 2 * H + (size_t)(2 * g) * R + hi) * D;
  const T* a2 = ctx + ((size_t)t * 2 * H + (size_t)(2 * g + 1) * R + hi) * D;
  float ss = 0.f;
  for (int c = lane; c < dv; c += WAVE) {
    const float o = to_f32(a1[c]) - lambda * to_f32(a2[c]);
    ss = fmaf(o, o, ss);
  }
  ss = wave_sum(ss);
  const float s = gain / sqrtf(ss / (float)dv + eps);
  T* o_row = out + ((size_t)t * H + h) * dv;
  for (int c = lane; c < dv; c += WAVE)
    from_f32(o_row + c, (to_f32(a1[c]) - lambda * to_f32(a2[c])) * s);
}

extern "C" int kappai_diff_combine(const void* ctx, void* out, int T, int H, int G, int dv, int D,
                                   float lambda, float eps, float gain, int is_bf16,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (H % G || dv > D || H > 65535) return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(diff_combine_kernel<bf16_t>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const bf16_t*)ctx, (bf16_t*)out, H, G, dv, D, lambda, eps, gain);
  else
    hipLaunchKernelGGL(diff_combine_kernel<float>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const float*)ctx, (float*)out, H, G, dv, D, lambda, eps, gain);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
