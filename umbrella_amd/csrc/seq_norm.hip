// Grouped RMS norm and the residual seams of the sequence-mixer stacks.  The residual stream is fp32; every sum of squares,
// factor and product is fp32; only the normed activations that feed a matrix product are rounded to the storage dtype.
//
//   group norm: a row of W values is cut into `groups` equal consecutive parts; each part is divided by its own
//   sqrt(mean(part^2) + eps); the whole row is multiplied by the weight.  groups == 1 is the plain RMS norm.
//
// One wave owns one (row, group): the three passes of the fused seam (sum y^2 | x += y f w_post, sum x^2 | h = x f' w_next)
// touch the same elements from the same lanes, so no barrier is needed and a row's result never depends on its neighbours.
#include "seq_common.h"

template <typename P>
__global__ __launch_bounds__(256) void group_norm_kernel(float* __restrict__ out_f32, typename El<P>::type* __restrict__ out_dt,
                                                         const float* __restrict__ x, const int* __restrict__ rows,
                                                         const typename El<P>::type* __restrict__ w, int W, int groups,
                                                         float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int grp = blockIdx.y * 4 + wave;
  if (grp >= groups) return;
  const int t = blockIdx.x, gs = W / groups;
  const float* xr = x + (long)(rows ? rows[t] : t) * W + (long)grp * gs;
  float ss = 0.f;
  for (int i = lane; i < gs; i += 64) { const float v = xr[i]; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)gs + eps);
  const long o = (long)t * W + (long)grp * gs;
  for (int i = lane; i < gs; i += 64) {
    const float v = xr[i] * f * ldf<P>(w + grp * gs + i);
    if (out_f32) out_f32[o + i] = v;
    if (out_dt) stf<P>(out_dt + o + i, v);
  }
}

template <typename P>
__global__ __launch_bounds__(256) void embed_norm_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                         const typename El<P>::type* __restrict__ embed,
                                                         const int* __restrict__ tokens, const typename El<P>::type* __restrict__ w,
                                                         int W, int V, int groups, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int grp = blockIdx.y * 4 + wave;
  if (grp >= groups) return;
  const int t = blockIdx.x, gs = W / groups;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  const typename El<P>::type* er = embed + (long)tok * W + (long)grp * gs;
  const long o = (long)t * W + (long)grp * gs;
  float ss = 0.f;
  for (int i = lane; i < gs; i += 64) { const float v = ldf<P>(er + i); x[o + i] = v; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)gs + eps);
  for (int i = lane; i < gs; i += 64) stf<P>(h + o + i, ldf<P>(er + i) * f * ldf<P>(w + grp * gs + i));
}

// values of one (row, group) held by a wave: lane owns elements lane + 64 j.  RV = 0: the group is longer than the register
// budget and is re-read from memory in every pass.
template <typename P, int RV>
__global__ __launch_bounds__(256) void resid_norm_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                         const float* __restrict__ y, const typename El<P>::type* __restrict__ w_post,
                                                         const typename El<P>::type* __restrict__ w_next, int W, int groups,
                                                         float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int grp = blockIdx.y * 4 + wave;
  if (grp >= groups) return;
  const int t = blockIdx.x, gs = W / groups;
  const long o = (long)t * W + (long)grp * gs;
  if constexpr (RV > 0) {
    // all loads of the pass are issued before the first use: one memory round trip per pass instead of one per element
    float yv[RV], xv[RV], wp[RV], wn[RV];
#pragma unroll
    for (int j = 0; j < RV; ++j) {
      const int i = lane + 64 * j, ic = i < gs ? i : gs - 1;
      yv[j] = y[o + ic];
      xv[j] = x[o + ic];
      wp[j] = ldf<P>(w_post + grp * gs + ic);
      wn[j] = w_next ? ldf<P>(w_next + grp * gs + ic) : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < RV; ++j) ss += lane + 64 * j < gs ? yv[j] * yv[j] : 0.f;
    ss = wave_sum(ss);
    const float f = 1.f / sqrtf(ss / (float)gs + eps);
    float s2 = 0.f;
#pragma unroll
    for (int j = 0; j < RV; ++j) {
      const int i = lane + 64 * j;
      xv[j] = xv[j] + yv[j] * f * wp[j];
      if (i < gs) { x[o + i] = xv[j]; s2 += xv[j] * xv[j]; }
    }
    if (!w_next) return;
    s2 = wave_sum(s2);
    const float f2 = 1.f / sqrtf(s2 / (float)gs + eps);
#pragma unroll
    for (int j = 0; j < RV; ++j) {
      const int i = lane + 64 * j;
      if (i < gs) stf<P>(h + o + i, xv[j] * f2 * wn[j]);
    }
  } else {
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) { const float v = y[o + i]; ss += v * v; }
    ss = wave_sum(ss);
    const float f = 1.f / sqrtf(ss / (float)gs + eps);
    float s2 = 0.f;
    for (int i = lane; i < gs; i += 64) {
      const float v = x[o + i] + y[o + i] * f * ldf<P>(w_post + grp * gs + i);
      x[o + i] = v;
      s2 += v * v;
    }
    if (!w_next) return;
    s2 = wave_sum(s2);
    const float f2 = 1.f / sqrtf(s2 / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) stf<P>(h + o + i, x[o + i] * f2 * ldf<P>(w_next + grp * gs + i));
  }
}

// ---- long groups (more than 16 elements per lane of one wave): a whole workgroup owns one (row, group), its 256 threads hold
// EPT elements each in registers, the two sums of squares go through LDS.  A decode step has few rows: one wave per row would
// leave a 4096-wide row to 64 lanes and three dependent passes over memory.
template <typename P, int EPT>
__global__ __launch_bounds__(256) void resid_norm_block_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                               const float* __restrict__ y,
                                                               const typename El<P>::type* __restrict__ w_post,
                                                               const typename El<P>::type* __restrict__ w_next, int W, int groups,
                                                               float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x, grp = blockIdx.y, gs = W / groups;
  const long o = (long)t * W + (long)grp * gs;
  float yv[EPT], xv[EPT], wp[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + 256 * e, ic = i < gs ? i : gs - 1;
    yv[e] = y[o + ic];
    xv[e] = x[o + ic];
    wp[e] = ldf<P>(w_post + grp * gs + ic);
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) ss += threadIdx.x + 256 * e < gs ? yv[e] * yv[e] : 0.f;
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)gs + eps);
  float s2 = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + 256 * e;
    xv[e] = xv[e] + yv[e] * f * wp[e];
    if (i < gs) { x[o + i] = xv[e]; s2 += xv[e] * xv[e]; }
  }
  {
    if (!w_next) return;
    s2 = block_sum<256>(s2, red);
    const float f2 = 1.f / sqrtf(s2 / (float)gs + eps);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      if (i < gs) stf<P>(h + o + i, xv[e] * f2 * ldf<P>(w_next + grp * gs + i));
    }
  }
}

template <typename P, int EPT>
__global__ __launch_bounds__(256) void group_norm_block_kernel(float* __restrict__ out_f32, typename El<P>::type* __restrict__ out_dt,
                                                               const float* __restrict__ x, const int* __restrict__ rows,
                                                               const typename El<P>::type* __restrict__ w, int W, int groups,
                                                               float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x, grp = blockIdx.y, gs = W / groups;
  const float* xr = x + (long)(rows ? rows[t] : t) * W + (long)grp * gs;
  float xv[EPT], ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + 256 * e;
    xv[e] = i < gs ? xr[i] : 0.f;
    ss += xv[e] * xv[e];
  }
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)gs + eps);
  const long o = (long)t * W + (long)grp * gs;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + 256 * e;
    if (i >= gs) continue;
    const float v = xv[e] * f * ldf<P>(w + grp * gs + i);
    if (out_f32) out_f32[o + i] = v;
    if (out_dt) stf<P>(out_dt + o + i, v);
  }
}

// The seam of a step of ONE token per sequence, followed by the next sublayer's causal convolution and its state update.
// Workgroup = (token, 256 channels); every workgroup of a token first sums the squares of the token's whole group of y by
// itself (a row is a few KiB: cheaper than a second launch), then each thread finishes one channel: x' = x + y f w_post,
// h = x' + sum_j w[c][j] x'(p - taps + 1 + j) with the earlier positions read from the sequence's state rows
// ((p - k) % (taps - 1)), and the state row of p overwritten with x' by the thread that read it.  The loads of the taps do not
// depend on one another (TAPS > 0: unrolled).
template <typename P, int TAPS>
__global__ __launch_bounds__(256) void seam_canon_step_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                              const float* __restrict__ y,
                                                              const typename El<P>::type* __restrict__ w_post,
                                                              const typename El<P>::type* __restrict__ canon,
                                                              float* __restrict__ state, const int* __restrict__ pos,
                                                              const int* __restrict__ slot, int W, int groups, float eps,
                                                              int taps_rt) {
  __shared__ float red[8];
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x, gs = W / groups;
  const int grp = (blockIdx.y * 256) / gs;                    // the workgroup's channels lie in one group
  const float* yr = y + (long)t * W + (long)grp * gs;
  float ss = 0.f;
#pragma unroll 8
  for (int i = threadIdx.x; i < gs; i += 256) { const float v = yr[i]; ss += v * v; }
  ss = block_sum<256>(ss, red);
  if (c >= W) return;
  const float f = 1.f / sqrtf(ss / (float)gs + eps);
  const int taps = TAPS > 0 ? TAPS : taps_rt, S = taps - 1;
  const int p = pos[t];
  float* st = state + (long)slot[t] * S * W + c;
  const typename El<P>::type* wc = canon + (long)c * taps;
  const float xn = x[(long)t * W + c] + y[(long)t * W + c] * f * ldf<P>(w_post + c);
  x[(long)t * W + c] = xn;
  float a = xn * (1.f + ldf<P>(wc + S));
  if constexpr (TAPS > 0) {
    float v[TAPS], wk[TAPS];
#pragma unroll
    for (int k = 1; k < TAPS; ++k) {
      v[k] = st[(long)((p - k >= 0 ? p - k : 0) % (TAPS - 1)) * W];
      wk[k] = ldf<P>(wc + (TAPS - 1) - k);
    }
#pragma unroll
    for (int k = 1; k < TAPS; ++k) a += p - k >= 0 ? wk[k] * v[k] : 0.f;
  } else {
    for (int k = 1; k <= S; ++k) {
      const float v = st[(long)((p - k >= 0 ? p - k : 0) % S) * W];
      a += p - k >= 0 ? ldf<P>(wc + S - k) * v : 0.f;
    }
  }
  stf<P>(h + (long)t * W + c, a);
  if (S > 0) st[(long)(p % S) * W] = xn;
}

static inline bool norm_args_ok(int T, int W, int groups) { return T >= 1 && W >= 1 && groups >= 1 && W % groups == 0; }

extern "C" int umb_seq_group_norm(float* out_f32, void* out_dt, const float* x, const int* rows, const void* w, int T, int W,
                                  int groups, float eps, int dtype, hipStream_t st) {
  if (!norm_args_ok(T, W, groups) || !x || !w || (!out_f32 && !out_dt)) return UMB_EINVAL;
  const int gs = W / groups;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    if (gs > 1024 && gs <= 2048)
      hipLaunchKernelGGL((group_norm_block_kernel<P, 8>), dim3(T, groups), dim3(256), 0, st, out_f32, (E*)out_dt, x, rows,
                         (const E*)w, W, groups, eps);
    else if (gs > 2048 && gs <= 8192)
      hipLaunchKernelGGL((group_norm_block_kernel<P, 32>), dim3(T, groups), dim3(256), 0, st, out_f32, (E*)out_dt, x, rows,
                         (const E*)w, W, groups, eps);
    else
      hipLaunchKernelGGL(group_norm_kernel<P>, dim3(T, (groups + 3) / 4), dim3(256), 0, st, out_f32, (E*)out_dt, x, rows,
                         (const E*)w, W, groups, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_seq_embed_norm(float* x, void* h, const void* embed, const int* tokens, const void* w, int T, int W, int V,
                                  int groups, float eps, int dtype, hipStream_t st) {
  if (!norm_args_ok(T, W, groups) || !x || !h || !embed || !tokens || !w || V < 1) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(embed_norm_kernel<P>, dim3(T, (groups + 3) / 4), dim3(256), 0, st, x, (E*)h, (const E*)embed, tokens,
                       (const E*)w, W, V, groups, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_seq_resid_norm(float* x, void* h, const float* y, const void* w_post, const void* w_next, int T, int W,
                                  int groups, float eps, int dtype, hipStream_t st) {
  if (!norm_args_ok(T, W, groups) || !x || !y || !w_post || (w_next && !h)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    const int per_lane = (W / groups + 63) / 64;
    const dim3 grid(T, (groups + 3) / 4);
    const int gs = W / groups;
    if (per_lane > 16 && gs <= 2048)
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 8>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)w_next, W, groups, eps);
    else if (per_lane > 16 && gs <= 8192)
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 32>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)w_next, W, groups, eps);
    else if (per_lane <= 4)
      hipLaunchKernelGGL((resid_norm_kernel<P, 4>), grid, dim3(256), 0, st, x, (E*)h, y, (const E*)w_post, (const E*)w_next, W,
                         groups, eps);
    else if (per_lane <= 16)
      hipLaunchKernelGGL((resid_norm_kernel<P, 16>), grid, dim3(256), 0, st, x, (E*)h, y, (const E*)w_post, (const E*)w_next, W,
                         groups, eps);
    else
      hipLaunchKernelGGL((resid_norm_kernel<P, 0>), grid, dim3(256), 0, st, x, (E*)h, y, (const E*)w_post, (const E*)w_next, W,
                         groups, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_seq_resid_canon_step_ok(int W, int groups) {
  return W >= 1 && groups >= 1 && W % groups == 0 && (groups == 1 || (W / groups) % 256 == 0);
}

extern "C" int umb_seq_resid_canon_step(float* x, void* h, const float* y, const void* w_post, const void* canon, float* state,
                                        const int* pos, const int* slot, int T, int W, int groups, int taps, float eps, int dtype,
                                        hipStream_t st) {
  if (!norm_args_ok(T, W, groups) || !x || !h || !y || !w_post || !canon || !pos || !slot || taps < 1 || (taps > 1 && !state) ||
      !umb_seq_resid_canon_step_ok(W, groups))
    return UMB_EINVAL;
  const dim3 grid(T, (W + 255) / 256);
#define SEAM_LAUNCH(TAPS)                                                                                                  \
  hipLaunchKernelGGL((seam_canon_step_kernel<P, TAPS>), grid, dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,             \
                     (const E*)canon, state, pos, slot, W, groups, eps, taps)
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    switch (taps) {
      case 2: SEAM_LAUNCH(2); break;
      case 3: SEAM_LAUNCH(3); break;
      case 4: SEAM_LAUNCH(4); break;
      case 5: SEAM_LAUNCH(5); break;
      default: SEAM_LAUNCH(0); break;
    }
  })
#undef SEAM_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
