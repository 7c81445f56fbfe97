// Gated linear attention: a [D][Dv] matrix state per (sequence, head), decayed per key channel and updated by an outer
// product at every token,
//     S_t = diag(alpha_t) S_(t-1) + k_t v_t^T        o_t = S_t^T q_t
// with alpha_t = sigmoid(W_a2 (W_a1 h_t) + b)^(1/tau) in (0, 1).  Everything here is fp32: the decay and its logarithm, the
// state, the products that enter it and the read-out.  The state lives in a slot array [slots][H][D][Dv] and is carried from
// step to step; a sequence whose first row is at position 0 starts from zero whatever its slot held before.
//
// scan kernel: one WAVE owns four value columns of one (sequence, head): lane (r = lane % 16, c = lane / 16) keeps rows
// r, r + 16, r + 32, ... of column c in registers, so the update is register-local and the read-out sum over rows is four
// xor-shuffles inside 16 lanes -- no LDS, no barrier, and the order of every sum is fixed by (D) alone.  The token loop is
// the only serial dimension; the next tokens' q / k / v / alpha are independent of the recurrence and are fetched ahead.
#include "seq_common.h"

template <typename P>
__global__ __launch_bounds__(256) void gla_decay_kernel(float* __restrict__ alpha, const float* __restrict__ proj, int ld,
                                                        int a_col, const typename El<P>::type* __restrict__ w_a2,
                                                        const typename El<P>::type* __restrict__ b_a2, int HD, int rank,
                                                        float inv_tau) {
  extern __shared__ float a_s[];
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < rank; i += 256) a_s[i] = proj[(long)t * ld + a_col + i];
  __syncthreads();
  for (int n = blockIdx.y * 256 + threadIdx.x; n < HD; n += gridDim.y * 256) {
    const typename El<P>::type* wr = w_a2 + (long)n * rank;
    float z = 0.f;
    for (int i = 0; i < rank; ++i) z += ldf<P>(wr + i) * a_s[i];
    if (b_a2) z += ldf<P>(b_a2 + n);
    alpha[(long)t * HD + n] = expf(log_sigmoidf_(z) * inv_tau);
  }
}

constexpr int GLA_MAXR = 16;     // rows per lane: D <= 256

template <int NR>
__global__ __launch_bounds__(64) void gla_scan_kernel(float* __restrict__ o, float* __restrict__ state,
                                                      const float* __restrict__ proj, int ld, const float* __restrict__ alpha,
                                                      const int* __restrict__ seq_slot, const int* __restrict__ seq_row0,
                                                      const int* __restrict__ seq_pos0, const int* __restrict__ seq_len, int H,
                                                      int D, int Dv, float qscale) {
  const int lane = threadIdx.x, r = lane & 15, c = blockIdx.x * 4 + (lane >> 4);
  const int h = blockIdx.y, b = blockIdx.z;
  const int n = seq_len[b];
  if (n <= 0) return;
  const bool c_ok = c < Dv;
  const int cc = c_ok ? c : 0;
  const int slot = seq_slot[b], row0 = seq_row0[b];
  float* sp = state + (((long)slot * H + h) * D) * Dv + cc;
  float S[NR];
  const bool fresh = seq_pos0[b] == 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = r + 16 * i;
    S[i] = (!fresh && d < D) ? sp[(long)d * Dv] : 0.f;
  }
  const int HD = H * D;
  const long qo = (long)h * D, ko = (long)HD + (long)h * D, vo = 2L * HD + (long)h * Dv + cc;
  for (int t = 0; t < n; ++t) {
    const float* pr = proj + (long)(row0 + t) * ld;
    const float* ar = alpha + (long)(row0 + t) * HD + (long)h * D;
    const float v = pr[vo];
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = r + 16 * i;
      if (d < D) {
        S[i] = ar[d] * S[i] + pr[ko + d] * v;
        acc += S[i] * (pr[qo + d] * qscale);
      }
    }
    acc += __shfl_xor(acc, 1, 64);
    acc += __shfl_xor(acc, 2, 64);
    acc += __shfl_xor(acc, 4, 64);
    acc += __shfl_xor(acc, 8, 64);
    if (r == 0 && c_ok) o[(long)(row0 + t) * (H * Dv) + (long)h * Dv + c] = acc;
  }
  if (c_ok) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = r + 16 * i;
      if (d < D) sp[(long)d * Dv] = S[i];
    }
  }
}

template <typename P>
__global__ __launch_bounds__(256) void gla_gate_kernel(typename El<P>::type* __restrict__ out, const float* __restrict__ o,
                                                       const float* __restrict__ proj, int ld, int g_col,
                                                       const typename El<P>::type* __restrict__ w, int T, int H, int Dv, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long th = (long)blockIdx.x * 4 + wave;           // (token, head)
  if (th >= (long)T * H) return;
  const int t = (int)(th / H), h = (int)(th % H);
  const float* orow = o + (long)t * H * Dv + (long)h * Dv;
  float ss = 0.f;
  for (int i = lane; i < Dv; i += 64) { const float v = orow[i]; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)Dv + eps);
  const float* gr = proj + (long)t * ld + g_col + (long)h * Dv;
  for (int i = lane; i < Dv; i += 64)
    stf<P>(out + (long)t * H * Dv + (long)h * Dv + i, orow[i] * f * ldf<P>(w + i) * siluf_(gr[i]));
}

extern "C" int umb_gla_decay(float* alpha, const float* proj, int ld, int a_col, const void* w_a2, const void* b_a2, int T, int HD,
                             int rank, float tau, int dtype, hipStream_t st) {
  if (T < 1 || HD < 1 || rank < 1 || rank > 8192 || !(tau > 0.f) || !alpha || !proj || !w_a2) return UMB_EINVAL;
  const int gy = (HD + 255) / 256 > 64 ? 64 : (HD + 255) / 256;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(gla_decay_kernel<P>, dim3(T, gy), dim3(256), rank * sizeof(float), st, alpha, proj, ld, a_col,
                       (const E*)w_a2, (const E*)b_a2, HD, rank, 1.f / tau);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_gla_scan(float* o, float* state, const float* proj, int ld, const float* alpha, const int* seq_slot,
                            const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv,
                            float qscale, hipStream_t st) {
  if (B < 1 || H < 1 || D < 1 || D > 16 * GLA_MAXR || Dv < 1 || !o || !state || !proj || !alpha) return UMB_EINVAL;
  const dim3 grid((Dv + 3) / 4, H, B);
  const int nr = (D + 15) / 16;
#define GLA_SCAN_CASE(NR)                                                                                                 \
  case NR:                                                                                                                \
    hipLaunchKernelGGL(gla_scan_kernel<NR>, grid, dim3(64), 0, st, o, state, proj, ld, alpha, seq_slot, seq_row0, seq_pos0, \
                       seq_len, H, D, Dv, qscale);                                                                        \
    break;
  switch (nr) {
    GLA_SCAN_CASE(1) GLA_SCAN_CASE(2) GLA_SCAN_CASE(3) GLA_SCAN_CASE(4) GLA_SCAN_CASE(5) GLA_SCAN_CASE(6) GLA_SCAN_CASE(7)
    GLA_SCAN_CASE(8) GLA_SCAN_CASE(9) GLA_SCAN_CASE(10) GLA_SCAN_CASE(11) GLA_SCAN_CASE(12) GLA_SCAN_CASE(13)
    GLA_SCAN_CASE(14) GLA_SCAN_CASE(15) GLA_SCAN_CASE(16)
    default: return UMB_EINVAL;
  }
#undef GLA_SCAN_CASE
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_gla_gate(void* out, const float* o, const float* proj, int ld, int g_col, const void* w, int T, int H, int Dv,
                            float eps, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || Dv < 1 || !out || !o || !proj || !w) return UMB_EINVAL;
  const long th = (long)T * H;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(gla_gate_kernel<P>, dim3((unsigned)((th + 3) / 4)), dim3(256), 0, st, (E*)out, o, proj, ld, g_col,
                       (const E*)w, T, H, Dv, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
