// General linear layer for the sequence-mixer models: out[T][N] = x[T][K] . W[N][K]^T + bias for ANY T, N, K, weights as
// stored (row-major [out][in], no repacking), 16-bit or fp32 storage, fp32 accumulation on the matrix pipe.
//
// Both operands are K-contiguous, so a lane's 8 consecutive K-elements of "its" row ARE its share of an MFMA operand:
//   v_mfma_f32_16x16x32_{bf16,f16}: A 16 rows x 32 k, lane (j = lane % 16, g = lane / 16) supplies row j, k 8g .. 8g+7
//   v_mfma_f32_16x16x4_f32 (true fp32, x8): the same 8 elements feed instruction i with element i of every lane, i.e. step i
//   multiplies k = 8g + i of A with k = 8g + i of B -- the pairing is what matters, the order inside the 32-k step is free.
// Weights are the A operand (rows = output features), tokens the B operand: lane l ends up with outputs
// (n = 4 (l / 16) + r, token = l % 16), r = 0..3.  Weights go HBM -> VGPR (every weight element is used by exactly one wave of
// a <= 64-token launch), as in the skinny GEMM of gemm.hip.
//
// A workgroup owns one 16-row output tile and up to 64 tokens; its four waves split K (wave w takes the 32-k steps w, w+4, ...)
// and their partial tiles are summed through LDS in wave order: the summation order of an output is a function of K alone,
// never of T or of the row's place in the batch.  K % 8 != 0 (or a tail) falls back to guarded element loads.
#include "seq_common.h"

template <typename P> struct Frag8 { u32x4 v; };
template <> struct Frag8<F32> { f32x4 lo, hi; };

template <typename P, bool VEC>
__device__ __forceinline__ Frag8<P> load8(const typename El<P>::type* __restrict__ row, bool ok, int k, int K) {
  Frag8<P> f;
  if constexpr (VEC) {                      // K % 8 == 0: k < K means the whole 8-group is inside, 16-byte aligned
    const bool in = ok && k < K;
    if constexpr (sizeof(typename El<P>::type) == 2) {
      f.v = in ? *reinterpret_cast<const u32x4*>(row + k) : u32x4{0u, 0u, 0u, 0u};
    } else {
      f.lo = in ? *reinterpret_cast<const f32x4*>(row + k) : f32x4{0.f, 0.f, 0.f, 0.f};
      f.hi = in ? *reinterpret_cast<const f32x4*>(row + k + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  } else {
    if constexpr (sizeof(typename El<P>::type) == 2) {
      unsigned e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = (ok && k + i < K) ? (unsigned)row[k + i] : 0u;
      f.v = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
    } else {
      float e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = (ok && k + i < K) ? row[k + i] : 0.f;
      f.lo = f32x4{e[0], e[1], e[2], e[3]};
      f.hi = f32x4{e[4], e[5], e[6], e[7]};
    }
  }
  return f;
}

template <typename P> __device__ __forceinline__ f32x4 mma8(const Frag8<P>& a, const Frag8<P>& b, f32x4 c) {
  return P::mfma(a.v, b.v, c);
}
template <> __device__ __forceinline__ f32x4 mma8<F32>(const Frag8<F32>& a, const Frag8<F32>& b, f32x4 c) {
#pragma unroll
  for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.lo[i], b.lo[i], c, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.hi[i], b.hi[i], c, 0, 0, 0);
  return c;
}

enum { EPI_F32 = 0, EPI_DT = 1, EPI_SILU_MUL = 2 };

// TT token tiles of 16 per workgroup; DUAL: a second weight matrix W2 = W + N * K (the "up" half) with its own accumulators
template <typename P, int TT, bool VEC, bool DUAL>
__global__ __launch_bounds__(256) void seq_linear_kernel(void* __restrict__ out_, const typename El<P>::type* __restrict__ x,
                                                         const typename El<P>::type* __restrict__ w,
                                                         const typename El<P>::type* __restrict__ bias, int T, int N, int K,
                                                         int epi) {
  typedef typename El<P>::type E;
  __shared__ float red[DUAL ? 2 : 1][4][TT][256];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int j = lane & 15, g = lane >> 4;
  const int n_row = blockIdx.x * 16 + j;
  const int t0 = blockIdx.y * (TT * 16);
  const bool n_ok = n_row < N;
  const E* wrow = w + (long)(n_ok ? n_row : 0) * K;
  const E* wrow2 = DUAL ? wrow + (long)N * K : wrow;
  const E* xrow[TT];
  bool t_ok[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int t = t0 + tt * 16 + j;
    t_ok[tt] = t < T;
    xrow[tt] = x + (long)(t_ok[tt] ? t : 0) * K;
  }
  f32x4 acc[TT], acc2[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) { acc[tt] = f32x4{0.f, 0.f, 0.f, 0.f}; acc2[tt] = f32x4{0.f, 0.f, 0.f, 0.f}; }

  constexpr int UN = TT == 1 ? 4 : 2;        // 32-k steps in flight per wave
  for (int k0 = wave * 32; k0 < K; k0 += 128 * UN) {
    Frag8<P> a[UN], a2[UN], b[UN][TT];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = k0 + u * 128 + g * 8;
      a[u] = load8<P, VEC>(wrow, n_ok, k, K);
      if constexpr (DUAL) a2[u] = load8<P, VEC>(wrow2, n_ok, k, K);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) b[u][tt] = load8<P, VEC>(xrow[tt], t_ok[tt], k, K);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        acc[tt] = mma8<P>(a[u], b[u][tt], acc[tt]);
        if constexpr (DUAL) acc2[tt] = mma8<P>(a2[u], b[u][tt], acc2[tt]);
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    *reinterpret_cast<f32x4*>(&red[0][wave][tt][lane * 4]) = acc[tt];
    if constexpr (DUAL) *reinterpret_cast<f32x4*>(&red[1][wave][tt][lane * 4]) = acc2[tt];
  }
  __syncthreads();
  // thread (l = tid / 4, r = tid % 4) finishes output (n = 4 (l / 16) + r, token = l % 16) of every token tile
  const int l = threadIdx.x >> 2, r = threadIdx.x & 3;
  const int n = blockIdx.x * 16 + 4 * (l >> 4) + r;
  if (n >= N) return;
  const float bv = bias ? ldf<P>(bias + n) : 0.f;
  const float bv2 = (DUAL && bias) ? ldf<P>(bias + N + n) : 0.f;
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int t = t0 + tt * 16 + (l & 15);
    if (t >= T) continue;
    float s = red[0][0][tt][threadIdx.x];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) s += red[0][ww][tt][threadIdx.x];
    s += bv;
    if constexpr (DUAL) {
      float u = red[1][0][tt][threadIdx.x];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) u += red[1][ww][tt][threadIdx.x];
      u += bv2;
      stf<P>(reinterpret_cast<E*>(out_) + (long)t * N + n, siluf_(s) * u);
    } else if (epi == EPI_DT) {
      stf<P>(reinterpret_cast<E*>(out_) + (long)t * N + n, s);
    } else {
      reinterpret_cast<float*>(out_)[(long)t * N + n] = s;
    }
  }
}

template <typename P, int TT, bool VEC>
static int launch_tt(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, hipStream_t st) {
  typedef typename El<P>::type E;
  const dim3 grid((N + 15) / 16, (T + TT * 16 - 1) / (TT * 16));
  if (epi == EPI_SILU_MUL)
    hipLaunchKernelGGL((seq_linear_kernel<P, TT, VEC, true>), grid, dim3(256), 0, st, out, (const E*)x, (const E*)w, (const E*)bias,
                       T, N, K, epi);
  else
    hipLaunchKernelGGL((seq_linear_kernel<P, TT, VEC, false>), grid, dim3(256), 0, st, out, (const E*)x, (const E*)w,
                       (const E*)bias, T, N, K, epi);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

template <typename P, bool VEC>
static int launch_vec(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, hipStream_t st) {
  if (T <= 16) return launch_tt<P, 1, VEC>(out, x, w, bias, T, N, K, epi, st);
  if (T <= 32) return launch_tt<P, 2, VEC>(out, x, w, bias, T, N, K, epi, st);
  return launch_tt<P, 4, VEC>(out, x, w, bias, T, N, K, epi, st);
}

extern "C" int umb_seq_linear(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, int dtype,
                              hipStream_t st) {
  if (T < 1 || N < 1 || K < 1 || epi < 0 || epi > 2 || !out || !x || !w) return UMB_EINVAL;
  if (epi == EPI_SILU_MUL) {
    if (N & 1) return UMB_EINVAL;
    N >>= 1;                                   // rows of each half
  }
  DISPATCH_SEQ_DTYPE(dtype, {
    if (K % 8 == 0) return launch_vec<P, true>(out, x, w, bias, T, N, K, epi, st);
    return launch_vec<P, false>(out, x, w, bias, T, N, K, epi, st);
  })
}
