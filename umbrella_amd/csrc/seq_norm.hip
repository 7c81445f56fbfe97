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
// CANON: the seam is followed by the causal convolution in front of the next sublayer, for a step of ONE token per sequence:
// h = x' + sum_j w[c][j] x'(p - taps + 1 + j), earlier positions read from the sequence's state rows ((p - k) % (taps - 1)),
// and the state row of p is overwritten with x' by the thread that read it -- seam, convolution and state update in one launch.
template <typename P, int EPT, bool CANON>
__global__ __launch_bounds__(256) void resid_norm_block_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                               const float* __restrict__ y,
                                                               const typename El<P>::type* __restrict__ w_post,
                                                               const typename El<P>::type* __restrict__ w_next, int W, int groups,
                                                               float eps, const typename El<P>::type* __restrict__ canon,
                                                               float* __restrict__ state, const int* __restrict__ pos,
                                                               const int* __restrict__ slot, int taps) {
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
  if constexpr (CANON) {
    const int p = pos[t], S = taps - 1;
    float* st = state + (long)slot[t] * S * W + (long)grp * gs;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      if (i >= gs) continue;
      const typename El<P>::type* wc = canon + ((long)grp * gs + i) * taps;
      float a = xv[e] * (1.f + ldf<P>(wc + S));
      for (int k = 1; k <= S; ++k) {
        const bool in = p - k >= 0;
        const float v = st[(long)((in ? p - k : 0) % S) * W + i];
        a += in ? ldf<P>(wc + S - k) * v : 0.f;
      }
      stf<P>(h + o + i, a);
      if (S > 0) st[(long)(p % S) * W + i] = xv[e];
    }
  } else {
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
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 8, false>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)w_next, W, groups, eps, (const E*)nullptr, (float*)nullptr, (const int*)nullptr,
                         (const int*)nullptr, 0);
    else if (per_lane > 16 && gs <= 8192)
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 32, false>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)w_next, W, groups, eps, (const E*)nullptr, (float*)nullptr, (const int*)nullptr,
                         (const int*)nullptr, 0);
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

extern "C" int umb_seq_resid_canon_step(float* x, void* h, const float* y, const void* w_post, const void* canon, float* state,
                                        const int* pos, const int* slot, int T, int W, int groups, int taps, float eps, int dtype,
                                        hipStream_t st) {
  if (!norm_args_ok(T, W, groups) || !x || !h || !y || !w_post || !canon || !pos || !slot || taps < 1 || (taps > 1 && !state) ||
      W / groups > 8192)
    return UMB_EINVAL;
  const int gs = W / groups;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    if (gs <= 1024)
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 4, true>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)nullptr, W, groups, eps, (const E*)canon, state, pos, slot, taps);
    else if (gs <= 2048)
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 8, true>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)nullptr, W, groups, eps, (const E*)canon, state, pos, slot, taps);
    else
      hipLaunchKernelGGL((resid_norm_block_kernel<P, 32, true>), dim3(T, groups), dim3(256), 0, st, x, (E*)h, y, (const E*)w_post,
                         (const E*)nullptr, W, groups, eps, (const E*)canon, state, pos, slot, taps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
