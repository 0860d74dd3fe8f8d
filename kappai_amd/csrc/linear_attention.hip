// Recurrences whose state is a matrix per head, S [d, dv] in float32 (a slot per request), with a
// decay per key channel:
//   gated linear attention   S <- diag(a) S + k v^T                      o = S^T q
//   gated delta rule         S <- diag(a) S; u = beta (v - S^T k); S <- S + k u^T;  o = S^T q
// and what stands around them: the short causal convolution with SiLU on the projections, the
// decays / unit vectors / step sizes in float32, and the per-head RMS norm with its gate.
//
// A column of S (one value channel) never meets another column, so the work of a (segment, head)
// is spread over lanes by value channel, and a column's d rows over KS neighbouring lanes whose
// partial dot products meet by lane exchanges.  Tokens of a segment are walked in order; a
// segment that starts at position 0 starts from zero, whatever the slot holds.
#include "common.h"

#define LA_THREADS 256

__device__ __forceinline__ float la_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float la_softplus(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// ---------------------------------------------------------------------------------------
// Short causal convolution per channel, then SiLU.  x [T, >= C] with a row stride, taps [C, n]
// (the last column meets the current token), state [slots, n - 1, C] float32: the last n - 1
// inputs of the request, oldest first.  One thread a (row, channel) for the outputs; a second
// kernel rewrites the state after the outputs are made.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(LA_THREADS) void conv_silu_kernel(
    const T* __restrict__ x, int x_stride, const float* __restrict__ taps, int n_taps,
    const float* __restrict__ state, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ seg_start,
    const int* __restrict__ seg_slot, int C, T* __restrict__ out) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * LA_THREADS + threadIdx.x;
  if (c >= C) return;
  const int seg = row_seg[t], first = seg_start[seg], pos = row_pos[t];
  const float* st = state + (size_t)seg_slot[seg] * (n_taps - 1) * C;
  float acc = 0.f;
  for (int j = 0; j < n_taps; ++j) {
    const int back = n_taps - 1 - j;          // how many tokens before this one
    if (back > pos) continue;                 // before the start of the sequence: zero
    float v;
    if (t - back >= first) v = to_f32(x[(size_t)(t - back) * x_stride + c]);
    else v = st[(size_t)(n_taps - 1 - (back - (t - first))) * C + c];
    acc = fmaf(taps[(size_t)c * n_taps + j], v, acc);
  }
  from_f32(out + (size_t)t * C + c, acc * la_sigmoid(acc));
}

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void conv_state_kernel(
    const T* __restrict__ x, int x_stride, int n_taps, float* __restrict__ state,
    const int* __restrict__ seg_start, const int* __restrict__ seg_pos0,
    const int* __restrict__ seg_slot, int C) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * LA_THREADS + threadIdx.x;
  if (c >= C) return;
  const int first = seg_start[seg], n = seg_start[seg + 1] - first, keep = n_taps - 1;
  float* st = state + (size_t)seg_slot[seg] * keep * C + c;
  const bool fresh = seg_pos0[seg] == 0;
  // entry i of the new history is input number n - keep + i of the segment; a negative number
  // reaches back into the old history (zero for a request that has just begun)
  float kept[16];
  for (int i = 0; i < keep; ++i) {
    const int src = n - keep + i;
    if (src >= 0) kept[i] = to_f32(x[(size_t)(first + src) * x_stride + c]);
    else kept[i] = fresh ? 0.f : st[(size_t)(keep + src) * C];
  }
  for (int i = 0; i < keep; ++i) st[(size_t)i * C] = kept[i];
}

extern "C" int kappai_conv_silu(const void* x, int x_stride, const float* taps, int n_taps,
                                float* state, const int* row_pos, const int* row_seg,
                                const int* seg_start, const int* seg_pos0, const int* seg_slot,
                                int T, int S, int C, void* out, int is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (n_taps < 1 || n_taps > 17 || S > 65535 || C > 65535 * LA_THREADS) return (int)hipErrorInvalidValue;
  const int bx = (C + LA_THREADS - 1) / LA_THREADS;
  if (is_bf16) {
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const bf16_t*)x, x_stride, taps, n_taps, state, row_pos, row_seg,
                       seg_start, seg_slot, C, (bf16_t*)out);
    if (n_taps > 1)
      hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                         (const bf16_t*)x, x_stride, n_taps, state, seg_start, seg_pos0, seg_slot,
                         C);
  } else {
    hipLaunchKernelGGL(conv_silu_kernel<float>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const float*)x, x_stride, taps, n_taps, state, row_pos, row_seg, seg_start,
                       seg_slot, C, (float*)out);
    if (n_taps > 1)
      hipLaunchKernelGGL(conv_state_kernel<float>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                         (const float*)x, x_stride, n_taps, state, seg_start, seg_pos0, seg_slot,
                         C);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// What enters the recurrence, in float32: a wave a (row, head).
//   qf, kf [T, Hk, d]   q and k (head h reads q/k head h / (H / Hk)), optionally made unit
//                       vectors x / sqrt(sum x^2 + unit_eps); q also times q_scale
//   af [T, H, d]        the decay exp(-rate[h] * softplus(sign * (z + z_bias)))
//   bf [T, H]           sigmoid(b) when b is given
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void recurrence_prep_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k, int k_stride,
    const T* __restrict__ z, int z_stride, const float* __restrict__ z_bias,
    const float* __restrict__ rate, float sign, const T* __restrict__ b, int b_stride, int H,
    int Hk, int d, int unit, float unit_eps, float q_scale, float* __restrict__ qf,
    float* __restrict__ kf, float* __restrict__ af, float* __restrict__ bf) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  if (h < Hk) {
    const T* qr = q + (size_t)t * q_stride + (size_t)h * d;
    const T* kr = k + (size_t)t * k_stride + (size_t)h * d;
    float sq = 0.f, sk = 0.f;
    for (int e = lane; e < d; e += WAVE) {
      const float a = to_f32(qr[e]), c = to_f32(kr[e]);
      sq = fmaf(a, a, sq);
      sk = fmaf(c, c, sk);
    }
    float fq = q_scale, fk = 1.f;
    if (unit) {
      fq = q_scale / sqrtf(wave_sum(sq) + unit_eps);
      fk = 1.0f / sqrtf(wave_sum(sk) + unit_eps);
    }
    for (int e = lane; e < d; e += WAVE) {
      qf[((size_t)t * Hk + h) * d + e] = to_f32(qr[e]) * fq;
      kf[((size_t)t * Hk + h) * d + e] = to_f32(kr[e]) * fk;
    }
  }
  const T* zr = z + (size_t)t * z_stride + (size_t)h * d;
  const float r = rate[h];
  for (int e = lane; e < d; e += WAVE) {
    const float zz = to_f32(zr[e]) + (z_bias ? z_bias[(size_t)h * d + e] : 0.f);
    af[((size_t)t * H + h) * d + e] = expf(-r * la_softplus(sign * zz));
  }
  if (b != nullptr && lane == 0)
    bf[(size_t)t * H + h] = la_sigmoid(to_f32(b[(size_t)t * b_stride + h]));
}

extern "C" int kappai_recurrence_prep(const void* q, int q_stride, const void* k, int k_stride,
                                      const void* z, int z_stride, const float* z_bias,
                                      const float* rate, float sign, const void* b, int b_stride,
                                      int T, int H, int Hk, int d, int unit, float unit_eps,
                                      float q_scale, float* qf, float* kf, float* af, float* bf,
                                      int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk || H > 65535 || d < 1) return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(recurrence_prep_kernel<bf16_t>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k, k_stride, (const bf16_t*)z,
                       z_stride, z_bias, rate, sign, (const bf16_t*)b, b_stride, H, Hk, d, unit,
                       unit_eps, q_scale, qf, kf, af, bf);
  else
    hipLaunchKernelGGL(recurrence_prep_kernel<float>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const float*)q, q_stride, (const float*)k, k_stride, (const float*)z,
                       z_stride, z_bias, rate, sign, (const float*)b, b_stride, H, Hk, d, unit,
                       unit_eps, q_scale, qf, kf, af, bf);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// The recurrence itself.  A wave takes 64 / KS value channels of one (segment, head); lane
// (c, s) keeps rows s * R .. s * R + R - 1 of column c in registers.  DELTA: the delta rule (needs
// beta), else the plain gated sum.  Loads of the next token are asked for before the current one
// is worked on.
// ---------------------------------------------------------------------------------------
#define LA_R 16

template <int KS>
__device__ __forceinline__ float ks_sum(float v) {
#pragma unroll
  for (int m = 1; m < KS; m <<= 1) v += __shfl_xor(v, m, WAVE);
  return v;
}

template <int KS, bool DELTA, typename TV>
__global__ __launch_bounds__(WAVE) void matrix_state_scan_kernel(
    const float* __restrict__ qf, const float* __restrict__ kf, const float* __restrict__ af,
    const float* __restrict__ bf, const TV* __restrict__ v, int v_stride,
    float* __restrict__ state, const int* __restrict__ seg_start,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int H, int Hk, int d,
    int dv, float* __restrict__ out) {
  constexpr int COLS = WAVE / KS;
  const int seg = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
  const int s = lane % KS, c = blockIdx.x * COLS + lane / KS;
  const bool col_ok = c < dv;
  const int cc = col_ok ? c : dv - 1;
  const int hk = h / (H / Hk);
  const int r0 = s * LA_R;
  const int first = seg_start[seg], last = seg_start[seg + 1];
  float* st = state + (((size_t)seg_slot[seg] * H + h) * d) * dv + cc;
  float S[LA_R];
  const bool carry = seg_pos0[seg] > 0;
#pragma unroll
  for (int r = 0; r < LA_R; ++r)
    S[r] = (carry && r0 + r < d) ? st[(size_t)(r0 + r) * dv] : 0.f;

  float qn[LA_R], kn[LA_R], an[LA_R], vn = 0.f, bn = 0.f;
  auto fetch = [&](int t) {
    const float* qr = qf + ((size_t)t * Hk + hk) * d + r0;
    const float* kr = kf + ((size_t)t * Hk + hk) * d + r0;
    const float* ar = af + ((size_t)t * H + h) * d + r0;
#pragma unroll
    for (int r = 0; r < LA_R; ++r) {
      const bool ok = r0 + r < d;
      qn[r] = ok ? qr[r] : 0.f;
      kn[r] = ok ? kr[r] : 0.f;
      an[r] = ok ? ar[r] : 0.f;
    }
    vn = to_f32(v[(size_t)t * v_stride + (size_t)h * dv + cc]);
    if (DELTA) bn = bf[(size_t)t * H + h];
  };
  if (first < last) fetch(first);
  for (int t = first; t < last; ++t) {
    float qc[LA_R], kc[LA_R], ac[LA_R];
#pragma unroll
    for (int r = 0; r < LA_R; ++r) { qc[r] = qn[r]; kc[r] = kn[r]; ac[r] = an[r]; }
    const float vc = vn, bc = bn;
    if (t + 1 < last) fetch(t + 1);
    float o = 0.f;
    if (DELTA) {
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < LA_R; ++r) {
        S[r] *= ac[r];
        dot = fmaf(S[r], kc[r], dot);
      }
      dot = ks_sum<KS>(dot);
      const float u = bc * (vc - dot);
#pragma unroll
      for (int r = 0; r < LA_R; ++r) {
        S[r] = fmaf(kc[r], u, S[r]);
        o = fmaf(S[r], qc[r], o);
      }
    } else {
#pragma unroll
      for (int r = 0; r < LA_R; ++r) {
        S[r] = fmaf(ac[r], S[r], kc[r] * vc);
        o = fmaf(S[r], qc[r], o);
      }
    }
    o = ks_sum<KS>(o);
    if (s == 0 && col_ok) out[(size_t)t * H * dv + (size_t)h * dv + c] = o;
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < LA_R; ++r)
      if (r0 + r < d) st[(size_t)(r0 + r) * dv] = S[r];
  }
}

template <int KS, bool DELTA>
static void scan_launch(const float* qf, const float* kf, const float* af, const float* bf,
                        const void* v, int v_stride, int v_is_bf16, float* state,
                        const int* seg_start, const int* seg_pos0, const int* seg_slot, int S,
                        int H, int Hk, int d, int dv, float* out, hipStream_t stream) {
  constexpr int COLS = WAVE / KS;
  dim3 grid((dv + COLS - 1) / COLS, H, S);
  if (v_is_bf16)
    hipLaunchKernelGGL((matrix_state_scan_kernel<KS, DELTA, bf16_t>), grid, dim3(WAVE), 0, stream,
                       qf, kf, af, bf, (const bf16_t*)v, v_stride, state, seg_start, seg_pos0,
                       seg_slot, H, Hk, d, dv, out);
  else
    hipLaunchKernelGGL((matrix_state_scan_kernel<KS, DELTA, float>), grid, dim3(WAVE), 0, stream,
                       qf, kf, af, bf, (const float*)v, v_stride, state, seg_start, seg_pos0,
                       seg_slot, H, Hk, d, dv, out);
}

extern "C" int kappai_matrix_state_scan(const float* qf, const float* kf, const float* af,
                                        const float* bf, const void* v, int v_stride,
                                        int v_is_bf16, float* state, const int* seg_start,
                                        const int* seg_pos0, const int* seg_slot, int T, int S,
                                        int H, int Hk, int d, int dv, int delta, float* out,
                                        hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk || H > 65535 || S > 65535 || d < 1 || d > 64 * LA_R || dv < 1)
    return (int)hipErrorInvalidValue;
  if (delta && bf == nullptr) return (int)hipErrorInvalidValue;
  int ks = 1;
  while (ks * LA_R < d) ks *= 2;
#define LA_CASE(KS_)                                                                            \
  case KS_:                                                                                     \
    if (delta)                                                                                  \
      scan_launch<KS_, true>(qf, kf, af, bf, v, v_stride, v_is_bf16, state, seg_start, seg_pos0, \
                             seg_slot, S, H, Hk, d, dv, out, stream);                           \
    else                                                                                        \
      scan_launch<KS_, false>(qf, kf, af, bf, v, v_stride, v_is_bf16, state, seg_start,         \
                              seg_pos0, seg_slot, S, H, Hk, d, dv, out, stream);                \
    break;
  switch (ks) {
    LA_CASE(1) LA_CASE(2) LA_CASE(4) LA_CASE(8) LA_CASE(16) LA_CASE(32) LA_CASE(64)
    default: return (int)hipErrorInvalidValue;
  }
#undef LA_CASE
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// Per head: o / sqrt(mean(o^2) + eps) * weight[dv] * gate, gate = silu(g) (kind 0) or sigmoid(g)
// (kind 1) of the projection g [T, >= H dv] with a row stride.  A wave a (row, head).
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void head_norm_gate_kernel(
    const float* __restrict__ o, const float* __restrict__ weight, float eps,
    const T* __restrict__ g, int g_stride, int gate_kind, int H, int dv, T* __restrict__ out) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += WAVE) ss = fmaf(orow[e], orow[e], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + (size_t)h * dv;
  for (int e = lane; e < dv; e += WAVE) {
    const float gv = to_f32(gr[e]);
    const float gate = gate_kind == 0 ? gv * la_sigmoid(gv) : la_sigmoid(gv);
    from_f32(out + ((size_t)t * H + h) * dv + e, orow[e] * inv * weight[e] * gate);
  }
}

extern "C" int kappai_head_norm_gate(const float* o, const float* weight, float eps, const void* g,
                                     int g_stride, int gate_kind, int T, int H, int dv, void* out,
                                     int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || H > 65535 || dv < 1 || gate_kind < 0 || gate_kind > 1)
    return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3(T, H), dim3(WAVE), 0, stream, o, weight,
                       eps, (const bf16_t*)g, g_stride, gate_kind, H, dv, (bf16_t*)out);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(T, H), dim3(WAVE), 0, stream, o, weight,
                       eps, (const float*)g, g_stride, gate_kind, H, dv, (float*)out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
