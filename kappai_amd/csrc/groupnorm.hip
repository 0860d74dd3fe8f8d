// RMS norm in groups with the residual sum in front of it, and the short causal convolution that
// a sublayer's input may pass before it is used ("h + conv(h)" per channel, its last taps - 1
// inputs kept per request).  Everything here is float32 arithmetic; only the rows that leave for
// a matrix product are rounded to the compute dtype.
#include "common.h"

#define GN_THREADS 256
#define CANON_MAX_TAPS 16

// resid[row] += delta[row] (bf16 or float rows, or n_part float partial sums added in order);
// then every group of D / groups consecutive values is divided by sqrt(mean(group^2) + eps) and
// the row multiplied by w.  `rows`: only these rows are normalised (the residual stays as it is).
// One block a row; the row lives in LDS between the two passes; a wave owns whole groups, so no
// sum crosses waves.
template <typename TO>
__global__ __launch_bounds__(GN_THREADS) void add_group_rmsnorm_kernel(
    float* __restrict__ resid, const void* __restrict__ delta, int delta_kind, int n_part,
    size_t part_stride, const float* __restrict__ w, float eps, int groups, int D,
    const int* __restrict__ rows, TO* __restrict__ out, int write_resid) {
  extern __shared__ float row[];          // D values, then `groups` scales
  float* scale = row + D;
  const int r_out = blockIdx.x;
  const int r = rows ? rows[r_out] : r_out;
  float* x = resid + (size_t)r * D;
  for (int i = threadIdx.x; i < D; i += GN_THREADS) {
    float v = x[i];
    if (delta_kind == 1) {
      v += bf16_to_f32(((const bf16_t*)delta)[(size_t)r * D + i]);
    } else if (delta_kind == 2) {
      const float* p = (const float*)delta + (size_t)r * D + i;
      for (int s = 0; s < n_part; ++s) v += p[s * part_stride];
    }
    row[i] = v;
    if (write_resid && delta_kind) x[i] = v;
  }
  __syncthreads();
  const int gs = D / groups;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  for (int g = wave; g < groups; g += GN_THREADS / WAVE) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += WAVE) {
      const float v = row[g * gs + i];
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) scale[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  TO* o = out + (size_t)r_out * D;
  for (int i = threadIdx.x; i < D; i += GN_THREADS)
    from_f32(o + i, row[i] * scale[i / gs] * w[i]);
}

extern "C" int kappai_add_group_rmsnorm(float* resid, const void* delta, int delta_kind,
                                        int n_part, int T, int D, const float* w, float eps,
                                        int groups, const int* rows, int n_rows, void* out,
                                        int out_is_bf16, int write_resid, hipStream_t stream) {
  const int n = rows ? n_rows : T;
  if (n <= 0) return 0;
  if (groups < 1 || D % groups || delta_kind < 0 || delta_kind > 2) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(D + groups) * sizeof(float);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
  const size_t ps = (size_t)T * D;
  if (out_is_bf16)
    hipLaunchKernelGGL(add_group_rmsnorm_kernel<bf16_t>, dim3(n), dim3(GN_THREADS), lds, stream,
                       resid, delta, delta_kind, n_part, ps, w, eps, groups, D, rows,
                       (bf16_t*)out, write_resid);
  else
    hipLaunchKernelGGL(add_group_rmsnorm_kernel<float>, dim3(n), dim3(GN_THREADS), lds, stream,
                       resid, delta, delta_kind, n_part, ps, w, eps, groups, D, rows, (float*)out,
                       write_resid);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// out[t, c] = h[t, c] + sum_j taps[c, j] * h(t - (n - 1) + j, c): an input before the row's
// segment comes from the request's state (the last n - 1 inputs, oldest first, [n - 1, D] a
// slot), an input before the sequence's start is zero.
template <typename TO>
__global__ __launch_bounds__(GN_THREADS) void canon_conv_kernel(
    const float* __restrict__ h, const float* __restrict__ taps, const float* __restrict__ state,
    const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ seg_start, const int* __restrict__ seg_slot, int n_taps, int D,
    TO* __restrict__ out) {
  const int t = blockIdx.x;
  const int seg = row_seg[t], pos = row_pos[t];
  const int local = t - seg_start[seg];
  const float* st = state + (size_t)seg_slot[seg] * (n_taps - 1) * D;
  for (int c = threadIdx.x; c < D; c += GN_THREADS) {
    const float* tw = taps + (size_t)c * n_taps;
    float acc = h[(size_t)t * D + c];
    for (int j = 0; j < n_taps; ++j) {
      const int back = n_taps - 1 - j;
      if (pos - back < 0) continue;
      const float v = (local - back >= 0) ? h[(size_t)(t - back) * D + c]
                                          : st[(size_t)(n_taps - 1 + local - back) * D + c];
      acc = fmaf(tw[j], v, acc);
    }
    from_f32(out + (size_t)t * D + c, acc);
  }
}

// The same for steps of many rows: a block takes CANON_ROWS rows in a row and a thread one
// channel of them, with the inputs of the rows before in registers (a row's input is read once
// and a bit, not once a tap).  A row near its segment's start takes what lies before the segment
// from the state, as above.  MAXT: the most taps the instance takes; the sums run in the same
// order as above.
#define CANON_ROWS 8

template <typename TO, int MAXT>
__global__ __launch_bounds__(GN_THREADS) void canon_conv_rows_kernel(
    const float* __restrict__ h, const float* __restrict__ taps, const float* __restrict__ state,
    const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ seg_start, const int* __restrict__ seg_slot, int n_taps, int D, int T,
    TO* __restrict__ out) {
  const int t0 = blockIdx.x * CANON_ROWS;
  const int c = blockIdx.y * GN_THREADS + threadIdx.x;
  if (c >= D) return;
  float twb[MAXT];            // the tap for the input b rows back
  float win[MAXT];            // win[b - 1]: the input b rows back in the batch (b = 1 ..)
  float cur[CANON_ROWS];
#pragma unroll
  for (int b = 0; b < MAXT; ++b) {
    twb[b] = b < n_taps ? taps[(size_t)c * n_taps + (n_taps - 1 - b)] : 0.f;
    const int tr = t0 - 1 - b;
    win[b] = (b < n_taps - 1 && tr >= 0) ? h[(size_t)tr * D + c] : 0.f;
  }
#pragma unroll
  for (int r = 0; r < CANON_ROWS; ++r) cur[r] = t0 + r < T ? h[(size_t)(t0 + r) * D + c] : 0.f;
#pragma unroll
  for (int r = 0; r < CANON_ROWS; ++r) {
    const int t = t0 + r;
    if (t < T) {
      const int seg = row_seg[t], pos = row_pos[t];
      const int local = t - seg_start[seg];
      float acc = cur[r];
#pragma unroll
      for (int b = MAXT - 1; b >= 1; --b) {
        if (b <= n_taps - 1 && pos - b >= 0) {
          const float v = local - b >= 0
                              ? win[b - 1]
                              : state[((size_t)seg_slot[seg] * (n_taps - 1) + (n_taps - 1 + local - b)) * D + c];
          acc = fmaf(twb[b], v, acc);
        }
      }
      acc = fmaf(twb[0], cur[r], acc);
      from_f32(out + (size_t)t * D + c, acc);
    }
#pragma unroll
    for (int b = MAXT - 1; b >= 1; --b) win[b] = win[b - 1];
    win[0] = cur[r];
  }
}

// The state after the step: the last n - 1 inputs of every segment's request, oldest first.  A
// thread owns a channel of a segment and reads what it keeps of the old state before it writes.
__global__ __launch_bounds__(GN_THREADS) void canon_state_kernel(
    const float* __restrict__ h, float* __restrict__ state, const int* __restrict__ seg_start,
    const int* __restrict__ seg_slot, int n_taps, int D) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * GN_THREADS + threadIdx.x;
  if (c >= D) return;
  const int first = seg_start[seg], L = seg_start[seg + 1] - first;
  float* st = state + (size_t)seg_slot[seg] * (n_taps - 1) * D;
  float keep[CANON_MAX_TAPS];
#pragma unroll
  for (int k = 0; k < CANON_MAX_TAPS; ++k) {
    if (k < n_taps - 1) {
      const int li = L + k - (n_taps - 1);
      keep[k] = li >= 0 ? h[(size_t)(first + li) * D + c] : st[(size_t)(L + k) * D + c];
    }
  }
#pragma unroll
  for (int k = 0; k < CANON_MAX_TAPS; ++k)
    if (k < n_taps - 1) st[(size_t)k * D + c] = keep[k];
}

extern "C" int kappai_canon_conv(const float* h, const float* taps, float* state,
                                 const int* row_pos, const int* row_seg, const int* seg_start,
                                 const int* seg_slot, int T, int S, int D, int n_taps, void* out,
                                 int out_is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (n_taps < 1 || n_taps > CANON_MAX_TAPS || S > 65535) return (int)hipErrorInvalidValue;
  const dim3 rows_grid((T + CANON_ROWS - 1) / CANON_ROWS, (D + GN_THREADS - 1) / GN_THREADS);
#define CANON_ROWS_LAUNCH(TT, MAXT_)                                                             \
  hipLaunchKernelGGL((canon_conv_rows_kernel<TT, MAXT_>), rows_grid, dim3(GN_THREADS), 0, stream,  \
                     h, taps, state, row_pos, row_seg, seg_start, seg_slot, n_taps, D, T, (TT*)out)
  if (T >= 8 * CANON_ROWS && rows_grid.y <= 65535) {
    // many rows: a block a run of rows
    if (out_is_bf16) {
      if (n_taps <= 4) CANON_ROWS_LAUNCH(bf16_t, 4); else CANON_ROWS_LAUNCH(bf16_t, CANON_MAX_TAPS);
    } else {
      if (n_taps <= 4) CANON_ROWS_LAUNCH(float, 4); else CANON_ROWS_LAUNCH(float, CANON_MAX_TAPS);
    }
  } else if (out_is_bf16)
    hipLaunchKernelGGL(canon_conv_kernel<bf16_t>, dim3(T), dim3(GN_THREADS), 0, stream, h, taps,
                       state, row_pos, row_seg, seg_start, seg_slot, n_taps, D, (bf16_t*)out);
  else
    hipLaunchKernelGGL(canon_conv_kernel<float>, dim3(T), dim3(GN_THREADS), 0, stream, h, taps,
                       state, row_pos, row_seg, seg_start, seg_slot, n_taps, D, (float*)out);
#undef CANON_ROWS_LAUNCH
  if (n_taps > 1)
    hipLaunchKernelGGL(canon_state_kernel, dim3((D + GN_THREADS - 1) / GN_THREADS, S),
                       dim3(GN_THREADS), 0, stream, h, state, seg_start, seg_slot, n_taps, D);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// A step of single rows (every segment one decoded token): residual sum, norm, convolution and
// the state's shift in one kernel, a block of 1024 threads a row (a thread has one or two columns
// of the usual widths: what it loads, it loads at once).  Row t is segment t; its history is all
// state.
#define GN_STEP_THREADS 1024
template <typename TO>
__global__ __launch_bounds__(GN_STEP_THREADS) void add_group_rmsnorm_canon_step_kernel(
    float* __restrict__ resid, const void* __restrict__ delta, int delta_kind, int n_part,
    size_t part_stride, const float* __restrict__ w, float eps, int groups, int D,
    const float* __restrict__ taps, float* __restrict__ state, const int* __restrict__ row_pos,
    const int* __restrict__ seg_slot, int n_taps, TO* __restrict__ out) {
  extern __shared__ float row[];
  float* scale = row + D;
  const int r = blockIdx.x;
  float* x = resid + (size_t)r * D;
  for (int i = threadIdx.x; i < D; i += GN_STEP_THREADS) {
    float v = x[i];
    if (delta_kind == 1) {
      v += bf16_to_f32(((const bf16_t*)delta)[(size_t)r * D + i]);
    } else if (delta_kind == 2) {
      const float* p = (const float*)delta + (size_t)r * D + i;
      for (int s = 0; s < n_part; ++s) v += p[s * part_stride];
    }
    row[i] = v;
    if (delta_kind) x[i] = v;
  }
  __syncthreads();
  const int gs = D / groups;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  for (int g = wave; g < groups; g += GN_STEP_THREADS / WAVE) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += WAVE) {
      const float v = row[g * gs + i];
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) scale[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  const int pos = row_pos[r];
  float* st = state + (size_t)seg_slot[r] * (n_taps - 1) * D;
  for (int c = threadIdx.x; c < D; c += GN_STEP_THREADS) {
    // state[k] is the input n - 1 - k places back; everything is asked for before it is used
    float keep[CANON_MAX_TAPS], tw[CANON_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < CANON_MAX_TAPS; ++k) {
      if (k < n_taps) tw[k] = taps[(size_t)c * n_taps + k];
      if (k < n_taps - 1) keep[k] = pos - (n_taps - 1 - k) >= 0 ? st[(size_t)k * D + c] : 0.f;
    }
    const float h = row[c] * scale[c / gs] * w[c];
    float acc = h;
#pragma unroll
    for (int k = 0; k < CANON_MAX_TAPS; ++k) {
      if (k < n_taps - 1) {
        acc = fmaf(tw[k], keep[k], acc);
        if (k > 0) st[(size_t)(k - 1) * D + c] = keep[k];      // one place older now
      } else if (k == n_taps - 1) {
        acc = fmaf(tw[k], h, acc);
      }
    }
    if (n_taps > 1) st[(size_t)(n_taps - 2) * D + c] = h;
    from_f32(out + (size_t)r * D + c, acc);
  }
}

// The same with everything a thread needs asked for at once: the residual and its update, and
// for the same columns the norm's weight, the taps and the state, so that the kernel makes one
// trip to memory before the sums and none after.  Widths up to GN_STEP_MAXC * 1024 columns and up
// to MAXT taps.
#define GN_STEP_MAXC 4

template <typename TO, int MAXT>
__global__ __launch_bounds__(GN_STEP_THREADS) void add_group_rmsnorm_canon_step_early_kernel(
    float* __restrict__ resid, const void* __restrict__ delta, int delta_kind, int n_part,
    size_t part_stride, const float* __restrict__ w, float eps, int groups, int D,
    const float* __restrict__ taps, float* __restrict__ state, const int* __restrict__ row_pos,
    const int* __restrict__ seg_slot, int n_taps, TO* __restrict__ out) {
  extern __shared__ float row[];
  float* scale = row + D;
  const int r = blockIdx.x;
  float* x = resid + (size_t)r * D;
  const int pos = row_pos[r];
  float* st = state + (size_t)seg_slot[r] * (n_taps - 1) * D;
  float xv[GN_STEP_MAXC], wv[GN_STEP_MAXC], keep[GN_STEP_MAXC][MAXT], tw[GN_STEP_MAXC][MAXT];
#pragma unroll
  for (int q = 0; q < GN_STEP_MAXC; ++q) {
    const int c = threadIdx.x + q * GN_STEP_THREADS;
    if (c < D) {
      float v = x[c];
      if (delta_kind == 1) {
        v += bf16_to_f32(((const bf16_t*)delta)[(size_t)r * D + c]);
      } else if (delta_kind == 2) {
        const float* p = (const float*)delta + (size_t)r * D + c;
        for (int s = 0; s < n_part; ++s) v += p[s * part_stride];
      }
      xv[q] = v;
      wv[q] = w[c];
#pragma unroll
      for (int k = 0; k < MAXT; ++k) {
        tw[q][k] = k < n_taps ? taps[(size_t)c * n_taps + k] : 0.f;
        keep[q][k] = (k < n_taps - 1 && pos - (n_taps - 1 - k) >= 0) ? st[(size_t)k * D + c] : 0.f;
      }
    }
  }
#pragma unroll
  for (int q = 0; q < GN_STEP_MAXC; ++q) {
    const int c = threadIdx.x + q * GN_STEP_THREADS;
    if (c < D) {
      row[c] = xv[q];
      if (delta_kind) x[c] = xv[q];
    }
  }
  __syncthreads();
  const int gs = D / groups;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  for (int g = wave; g < groups; g += GN_STEP_THREADS / WAVE) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += WAVE) {
      const float v = row[g * gs + i];
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) scale[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < GN_STEP_MAXC; ++q) {
    const int c = threadIdx.x + q * GN_STEP_THREADS;
    if (c < D) {
      const float h = xv[q] * scale[c / gs] * wv[q];
      float acc = h;
#pragma unroll
      for (int k = 0; k < MAXT; ++k) {
        if (k < n_taps - 1) {
          acc = fmaf(tw[q][k], keep[q][k], acc);
          if (k > 0) st[(size_t)(k - 1) * D + c] = keep[q][k];
        } else if (k == n_taps - 1) {
          acc = fmaf(tw[q][k], h, acc);
        }
      }
      if (n_taps > 1) st[(size_t)(n_taps - 2) * D + c] = h;
      from_f32(out + (size_t)r * D + c, acc);
    }
  }
}

extern "C" int kappai_add_group_rmsnorm_canon_step(float* resid, const void* delta, int delta_kind,
                                                   int n_part, int T, int D, const float* w,
                                                   float eps, int groups, const float* taps,
                                                   float* state, const int* row_pos,
                                                   const int* seg_slot, int n_taps, void* out,
                                                   int out_is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (groups < 1 || D % groups || delta_kind < 0 || delta_kind > 2 || n_taps < 1 ||
      n_taps > CANON_MAX_TAPS)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(D + groups) * sizeof(float);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
  const size_t ps = (size_t)T * D;
  if (D <= GN_STEP_MAXC * GN_STEP_THREADS && n_taps <= 4) {
    if (out_is_bf16)
      hipLaunchKernelGGL((add_group_rmsnorm_canon_step_early_kernel<bf16_t, 4>), dim3(T),
                         dim3(GN_STEP_THREADS), lds, stream, resid, delta, delta_kind, n_part, ps, w,
                         eps, groups, D, taps, state, row_pos, seg_slot, n_taps, (bf16_t*)out);
    else
      hipLaunchKernelGGL((add_group_rmsnorm_canon_step_early_kernel<float, 4>), dim3(T),
                         dim3(GN_STEP_THREADS), lds, stream, resid, delta, delta_kind, n_part, ps, w,
                         eps, groups, D, taps, state, row_pos, seg_slot, n_taps, (float*)out);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  if (out_is_bf16)
    hipLaunchKernelGGL(add_group_rmsnorm_canon_step_kernel<bf16_t>, dim3(T), dim3(GN_STEP_THREADS), lds,
                       stream, resid, delta, delta_kind, n_part, ps, w, eps, groups, D, taps, state,
                       row_pos, seg_slot, n_taps, (bf16_t*)out);
  else
    hipLaunchKernelGGL(add_group_rmsnorm_canon_step_kernel<float>, dim3(T), dim3(GN_STEP_THREADS), lds,
                       stream, resid, delta, delta_kind, n_part, ps, w, eps, groups, D, taps, state,
                       row_pos, seg_slot, n_taps, (float*)out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// x[t] = x[t] * scale + table[row_pos[t]]: the embedding's scale and a learned row per position.
template <typename TT>
__global__ __launch_bounds__(GN_THREADS) void scale_add_positions_kernel(
    float* __restrict__ x, float scale, const TT* __restrict__ table, const int* __restrict__ row_pos,
    int D, int n_positions) {
  const int t = blockIdx.x;
  // (the host refuses a step past the table; a row of a warm-up run may carry any position)
  const TT* p = table + (size_t)min(max(row_pos[t], 0), n_positions - 1) * D;
  for (int i = threadIdx.x; i < D; i += GN_THREADS)
    x[(size_t)t * D + i] = fmaf(x[(size_t)t * D + i], scale, to_f32(p[i]));
}

extern "C" int kappai_scale_add_positions(float* x, float scale, const void* table,
                                          int table_is_bf16, const int* row_pos, int T, int D,
                                          int n_positions, hipStream_t stream) {
  if (T <= 0) return 0;
  if (n_positions < 1) return (int)hipErrorInvalidValue;
  if (table_is_bf16)
    hipLaunchKernelGGL(scale_add_positions_kernel<bf16_t>, dim3(T), dim3(GN_THREADS), 0, stream, x,
                       scale, (const bf16_t*)table, row_pos, D, n_positions);
  else
    hipLaunchKernelGGL(scale_add_positions_kernel<float>, dim3(T), dim3(GN_THREADS), 0, stream, x,
                       scale, (const float*)table, row_pos, D, n_positions);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
