// Scaled embedding lookup and the causal convolution over time in front of a sublayer.
//
// The convolution works on the fp32 residual stream, channel by channel:
//     h[t][c] = x[t][c] + sum_{j < taps} w[c][j] * x(p - taps + 1 + j)[c]          (p = the token's position; j = taps - 1 is itself)
// A position before the sequence's start contributes zero.  A position of an earlier step comes from the sequence's state,
// fp32 [slots][taps - 1][W], where the input at position p lives in row p % (taps - 1): a step of any length only overwrites
// the rows of its own last taps - 1 positions, so shorter steps keep what earlier ones left.  A sequence that starts at
// position 0 never reads its slot's state: nothing has to be cleared when a slot is handed out again.
//
// Within a step the rows of a sequence are contiguous and in position order, so position p - k is row t - k whenever that
// row belongs to the same slot.  The convolution kernel only reads the state; the update kernel runs after it.  For steps of
// one token per sequence both happen in one kernel: the thread that reads a channel's rows is the one that overwrites the
// oldest of them.
#include "seq_common.h"

template <typename P>
__global__ __launch_bounds__(256) void embed_kernel(float* __restrict__ x, const typename El<P>::type* __restrict__ embed,
                                                    const int* __restrict__ tokens, float scale, int W, int V) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  for (int i = threadIdx.x; i < W; i += 256) x[(long)t * W + i] = ldf<P>(embed + (long)tok * W + i) * scale;
}

// FUSED: T == number of sequences, one token each; the state row of the token's own position is written after the reads.
// One thread per (token, channel); the loads of the taps do not depend on one another.
template <typename P, bool FUSED>
__global__ __launch_bounds__(256) void canon_conv_kernel(typename El<P>::type* __restrict__ h, const float* __restrict__ x,
                                                         const typename El<P>::type* __restrict__ w, float* __restrict__ state,
                                                         const int* __restrict__ pos, const int* __restrict__ slot, int W,
                                                         int taps) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int p = pos[t], sl = slot[t], S = taps - 1;
  const float own = x[(long)t * W + c];
  float a = own * (1.f + ldf<P>(w + (long)c * taps + S));
  for (int k = 1; k <= S; ++k) {
    const bool in = p - k >= 0;
    const bool here = !FUSED && t - k >= 0 && slot[t - k < 0 ? 0 : t - k] == sl;
    const float* src = here ? x + (long)(t - k) * W + c : state + ((long)sl * S + (in ? p - k : 0) % S) * W + c;
    const float v = *src;
    a += in ? ldf<P>(w + (long)c * taps + S - k) * v : 0.f;
  }
  stf<P>(h + (long)t * W + c, a);
  if (FUSED && S > 0) state[((long)sl * S + p % S) * W + c] = own;
}

__global__ __launch_bounds__(256) void canon_update_kernel(float* __restrict__ state, const float* __restrict__ x,
                                                           const int* __restrict__ seq_slot, const int* __restrict__ seq_row0,
                                                           const int* __restrict__ seq_pos0, const int* __restrict__ seq_len,
                                                           int W, int S) {
  const int b = blockIdx.x, k = blockIdx.y;         // the k-th last position of sequence b's step
  const int n = seq_len[b];
  if (k >= n) return;
  const int p = seq_pos0[b] + n - 1 - k;
  const long row = seq_row0[b] + n - 1 - k;
  float* dst = state + ((long)seq_slot[b] * S + p % S) * W;
  for (int c = threadIdx.x; c < W; c += 256) dst[c] = x[row * W + c];
}

extern "C" int umb_seq_embed(float* x, const void* embed, const int* tokens, float scale, int T, int W, int V, int dtype,
                             hipStream_t st) {
  if (T < 1 || W < 1 || V < 1 || !x || !embed || !tokens) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(embed_kernel<P>, dim3(T), dim3(256), 0, st, x, (const E*)embed, tokens, scale, W, V);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_canon_conv(void* h, const float* x, const void* w, const float* state, const int* pos, const int* slot, int T,
                              int W, int taps, int dtype, hipStream_t st) {
  if (T < 1 || W < 1 || taps < 1 || !h || !x || !w || !pos || !slot || (taps > 1 && !state)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL((canon_conv_kernel<P, false>), dim3(T, (W + 255) / 256), dim3(256), 0, st, (E*)h, x, (const E*)w, const_cast<float*>(state),
                       pos, slot, W, taps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_canon_update(float* state, const float* x, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                                const int* seq_len, int B, int W, int taps, hipStream_t st) {
  if (B < 1 || W < 1 || taps < 1 || !x || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len || (taps > 1 && !state))
    return UMB_EINVAL;
  if (taps == 1) return UMB_OK;
  hipLaunchKernelGGL(canon_update_kernel, dim3(B, taps - 1), dim3(256), 0, st, state, x, seq_slot, seq_row0, seq_pos0, seq_len, W,
                     taps - 1);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_canon_step(void* h, const float* x, const void* w, float* state, const int* pos, const int* slot, int T, int W,
                              int taps, int dtype, hipStream_t st) {
  if (T < 1 || W < 1 || taps < 1 || !h || !x || !w || !pos || !slot || (taps > 1 && !state)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL((canon_conv_kernel<P, true>), dim3(T, (W + 255) / 256), dim3(256), 0, st, (E*)h, x, (const E*)w, state, pos, slot, W, taps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
