// Sliding-window attention with mean-pooled blocks behind the window, sigmoid weights (no softmax, nothing normalised over
// keys), over a PAGED key/value store shared by many sequences.
//
//   position i sees   tokens j with 0 <= i - j < window
//              and    blocks b (positions b pool .. b pool + pool - 1) with b pool + pool - 1 <= i - window,
//                     each through ONE key = mean of its cached keys and ONE value = mean of its cached values;
//   tokens that left the window but whose block is not complete behind it are not seen at all.
//   weight of a visible key = sigmoid(q.k * scale + bias[head]);  out = sigmoid(gate) * sum weight * v.
//
// Keys are cached AFTER rotation and unit-RMS scaling, values are the key projection as it came out of the matrix product
// (before rotation and scaling): one projection serves both.  Rotary: interleaved pairs (2i, 2i+1) of the first rot_dims
// features turn by angle pos * freq[i], computed in fp32 with the full-range sincosf.
//
// Store: pages of `page` tokens handed out by the host-side manager; per layer K, V [pages][G][page][D] in the storage
// dtype and pooled K, V [pages][G][ceil(page / pool)][D] in fp32.  A pooled block lives in the page of its last position, so
// it is born complete (all its tokens are cached by then, in this or earlier pages of the sequence) and dies with the
// sequence.  The pooled mean is always taken over the cached (rounded) values in position order: the same numbers whether
// the tokens arrived in one step or one by one.
//
// Because the weights are not normalised there is no running maximum and no rescaling: a query's output is a plain sum, and
// each (token, head) sums its keys in position order per lane column -- independent of the batch and of how the prompt was cut.
#include "seq_common.h"

// ---- rotary + unit RMS + cache append.  One wave per (token, head slot); head slots 0..H-1 are queries, H..H+G-1 keys.
template <typename P>
__global__ __launch_bounds__(256) void pwa_prep_kernel(float* __restrict__ q, UmbPagedKV kv, const float* __restrict__ proj, int ld,
                                                       const int* __restrict__ pos, const int* __restrict__ slot,
                                                       const float* __restrict__ freq, int T, int H, int G, int D, int rot_dims,
                                                       float eps) {
  typedef typename El<P>::type E;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long id = (long)blockIdx.x * 4 + wave;
  if (id >= (long)T * (H + G)) return;
  const int t = (int)(id / (H + G)), hs = (int)(id % (H + G));
  const bool is_q = hs < H;
  const float* src = proj + (long)t * ld + (is_q ? (long)hs * D : (long)H * D + (long)(hs - H) * D);
  const int p = pos[t];
  const float pf = (float)p;
  float* qd = is_q ? q + (long)t * H * D + (long)hs * D : nullptr;
  E* kd = nullptr;
  E* vd = nullptr;
  if (!is_q) {
    const long off = pkv_tok(kv, slot[t], p, hs - H, G, D);
    kd = reinterpret_cast<E*>(kv.k) + off;
    vd = reinterpret_cast<E*>(kv.v) + off;
  }
  // pass 1: rotate pairs, sum of squares (each lane owns whole pairs: features 2m, 2m+1 for m = lane, lane + 64, ...)
  float ss = 0.f;
  const int pairs = (D + 1) / 2;
  for (int m = lane; m < pairs; m += 64) {
    const int d0 = 2 * m, d1 = 2 * m + 1;
    float u = src[d0], v = d1 < D ? src[d1] : 0.f;
    if (!is_q) { stf<P>(vd + d0, u); if (d1 < D) stf<P>(vd + d1, v); }
    if (d1 < rot_dims) {
      float sn, cs;
      sincosf(pf * freq[m], &sn, &cs);
      const float ru = u * cs - v * sn, rv = v * cs + u * sn;
      u = ru; v = rv;
    }
    ss += u * u + (d1 < D ? v * v : 0.f);
  }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)D + eps);
  for (int m = lane; m < pairs; m += 64) {
    const int d0 = 2 * m, d1 = 2 * m + 1;
    float u = src[d0], v = d1 < D ? src[d1] : 0.f;
    if (d1 < rot_dims) {
      float sn, cs;
      sincosf(pf * freq[m], &sn, &cs);
      const float ru = u * cs - v * sn, rv = v * cs + u * sn;
      u = ru; v = rv;
    }
    if (is_q) { qd[d0] = u * f; if (d1 < D) qd[d1] = v * f; }
    else { stf<P>(kd + d0, u * f); if (d1 < D) stf<P>(kd + d1, v * f); }
  }
}

// ---- pooled blocks completed by this step: grid (block-in-step, sequence, kv head), one wave each
template <typename P>
__global__ __launch_bounds__(64) void pwa_pool_kernel(UmbPagedKV kv, const int* __restrict__ seq_slot,
                                                      const int* __restrict__ seq_pos0, const int* __restrict__ seq_len, int G,
                                                      int D, int pool) {
  typedef typename El<P>::type E;
  const int b = blockIdx.y, g = blockIdx.z, lane = threadIdx.x;
  const int p0 = seq_pos0[b], n = seq_len[b];
  if (n <= 0) return;
  // blocks whose last position e = blk pool + pool - 1 lies in [p0, p0 + n): blk >= ceil((p0 - pool + 1) / pool) = p0 / pool
  const int first = p0 / pool;
  const int blk = first + blockIdx.x;
  const int e = blk * pool + pool - 1;
  if (e >= p0 + n) return;
  const int slot = seq_slot[b];
  const long dst = pkv_blk(kv, slot, blk, pool, g, G, D);
  const float inv = 1.f / (float)pool;
  for (int d = lane; d < D; d += 64) {
    float sk = 0.f, sv = 0.f;
    for (int j = 0; j < pool; ++j) {
      const long off = pkv_tok(kv, slot, blk * pool + j, g, G, D) + d;
      sk += ldf<P>(reinterpret_cast<const E*>(kv.k) + off);
      sv += ldf<P>(reinterpret_cast<const E*>(kv.v) + off);
    }
    kv.kp[dst + d] = sk * inv;
    kv.vp[dst + d] = sv * inv;
  }
}

// ---- attention.  Workgroup = (token, RH query heads of one key/value group): the heads of a group read the same keys and
// values, so one pass over the keys serves all of them.  The NW waves take the 64-key rounds w, w + NW, ... of the key list
// (pooled blocks first, then the window's tokens, both in position order) and their partial sums are added through LDS in
// wave order -- which keys land in which wave depends on the query's position alone, never on the batch or on how the prompt
// was cut.  Score phase: lane = key, 16-byte loads along the key's row against the queries held in LDS.  Value phase:
// lane = value column, the round's weights broadcast one key at a time.
constexpr int PWA_MAXC = 4;      // value columns per lane: D <= 256

template <typename P, int RH, int NC, int NW>
__global__ __launch_bounds__(NW * 64) void pwa_attend_kernel(typename El<P>::type* __restrict__ out, const float* __restrict__ q,
                                                         UmbPagedKV kv, const float* __restrict__ proj, int ld, int gate_col,
                                                         const typename El<P>::type* __restrict__ pos_bias,
                                                         const int* __restrict__ pos, const int* __restrict__ slot_, int T, int H,
                                                         int G, int D, int window, int pool, float scale) {
  typedef typename El<P>::type E;
  extern __shared__ float lds[];
  constexpr int PWA_KB = 8;   // keys whose value rows are in flight together (32 measured 3x slower at 16 waves: registers)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Dp = (D + 3) & ~3;
  float* q_s = lds;                                          // [RH][Dp] queries; later [NW][RH][Dp] partial outputs
  float* w_s = lds + NW * RH * Dp + wave * (RH * 64 + 128);  // per wave: [RH][64] weights, [64] 64-bit offsets
  long* off_s = reinterpret_cast<long*>(w_s + RH * 64);
  const int t = blockIdx.x, h0 = blockIdx.y * RH;
  const int g = h0 / (H / G);
  const int i = pos[t], slot = slot_[t];
  for (int x = threadIdx.x; x < RH * D; x += NW * 64) q_s[(x / D) * Dp + x % D] = q[(long)t * H * D + (long)h0 * D + x];
  float bias[RH];
#pragma unroll
  for (int r = 0; r < RH; ++r) bias[r] = pos_bias ? ldf<P>(pos_bias + h0 + r) : 0.f;
  __syncthreads();
  const int j_lo = i - window + 1 > 0 ? i - window + 1 : 0;
  const int n_blk = i - window + 1 >= pool ? (i - window + 1) / pool : 0;
  const int n_keys = n_blk + (i - j_lo + 1);
  const bool vec = (D & 7) == 0;
  float acc[RH][NC];
#pragma unroll
  for (int r = 0; r < RH; ++r)
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[r][c] = 0.f;
  for (int base = wave * 64; base < n_keys; base += NW * 64) {
    const int kx = base + lane;
    float s[RH];
#pragma unroll
    for (int r = 0; r < RH; ++r) s[r] = 0.f;
    long off = 0;
    bool pooled = false;
    if (kx < n_keys) {
      pooled = kx < n_blk;
      off = pooled ? pkv_blk(kv, slot, kx, pool, g, G, D) : pkv_tok(kv, slot, j_lo + (kx - n_blk), g, G, D);
      if (pooled) {
        const float* kr = kv.kp + off;
        if ((D & 3) == 0) {
          for (int d = 0; d < D; d += 32) {              // eight 16-byte loads in flight, then their 32 x RH products
            f32x4 kk[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) kk[u] = *reinterpret_cast<const f32x4*>(kr + (d + 4 * u < D ? d + 4 * u : 0));
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              if (d + 4 * u >= D) break;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
#pragma unroll
                for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + d + 4 * u + e] * kk[u][e];
              }
            }
          }
        } else {
          for (int d = 0; d < D; ++d) {
            const float kd = kr[d];
#pragma unroll
            for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + d] * kd;
          }
        }
      } else {
        const E* kr = reinterpret_cast<const E*>(kv.k) + off;
        bool done = false;
        if constexpr (sizeof(E) == 2) {
          if (vec) {
            for (int d = 0; d < D; d += 64) {            // eight 16-byte loads in flight, then their 64 x RH products
              u32x4 kk[8];
#pragma unroll
              for (int u = 0; u < 8; ++u) kk[u] = *reinterpret_cast<const u32x4*>(kr + (d + 8 * u < D ? d + 8 * u : 0));
#pragma unroll
              for (int u = 0; u < 8; ++u) {
                if (d + 8 * u >= D) break;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const float k0 = lo_f<P>(kk[u][e]), k1 = hi_f<P>(kk[u][e]);
                  const int dd = d + 8 * u + 2 * e;
#pragma unroll
                  for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + dd] * k0 + q_s[r * Dp + dd + 1] * k1;
                }
              }
            }
            done = true;
          }
        }
        if (!done) {
          for (int d = 0; d < D; ++d) {
            const float kd = ldf<P>(kr + d);
#pragma unroll
            for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + d] * kd;
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RH; ++r) w_s[r * 64 + lane] = kx < n_keys ? 1.f / (1.f + expf(-(s[r] * scale + bias[r]))) : 0.f;
    off_s[lane] = pooled ? ~off : off;            // pooled entries are flagged by the complement (off >= 0 always)
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int cnt = n_keys - base < 64 ? n_keys - base : 64;
    // value rows: PWA_KB keys are fetched together, then used.  The round's keys are pooled entries first (fp32), then
    // tokens (storage dtype): two loops, so that no load sits behind a branch on the entry's kind; indices past the end are
    // clamped and weighted 0.
    const int cntp = n_blk - base < 0 ? 0 : (n_blk - base < cnt ? n_blk - base : cnt);
    int dcl[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) dcl[c] = lane + 64 * c < D ? lane + 64 * c : D - 1;
    for (int j0 = 0; j0 < cntp; j0 += PWA_KB) {
      float vv[PWA_KB][NC];
#pragma unroll
      for (int u = 0; u < PWA_KB; ++u) {
        const long oj = ~off_s[j0 + u < cntp ? j0 + u : cntp - 1];
#pragma unroll
        for (int c = 0; c < NC; ++c) vv[u][c] = kv.vp[oj + dcl[c]];
      }
#pragma unroll
      for (int u = 0; u < PWA_KB; ++u) {
#pragma unroll
        for (int r = 0; r < RH; ++r) {
          const float wj = j0 + u < cntp ? w_s[r * 64 + j0 + u] : 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) acc[r][c] += wj * vv[u][c];
        }
      }
    }
    for (int j0 = cntp; j0 < cnt; j0 += PWA_KB) {
      float vv[PWA_KB][NC];
#pragma unroll
      for (int u = 0; u < PWA_KB; ++u) {
        const long oj = off_s[j0 + u < cnt ? j0 + u : cnt - 1];
#pragma unroll
        for (int c = 0; c < NC; ++c) vv[u][c] = ldf<P>(reinterpret_cast<const E*>(kv.v) + oj + dcl[c]);
      }
#pragma unroll
      for (int u = 0; u < PWA_KB; ++u) {
#pragma unroll
        for (int r = 0; r < RH; ++r) {
          const float wj = j0 + u < cnt ? w_s[r * 64 + j0 + u] : 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) acc[r][c] += wj * vv[u][c];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();                                  // every wave is done with the queries: their LDS becomes the partials
#pragma unroll
  for (int r = 0; r < RH; ++r)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < D) lds[(wave * RH + r) * Dp + d] = acc[r][c];
    }
  __syncthreads();
  for (int x = threadIdx.x; x < RH * D; x += NW * 64) {
    const int r = x / D, d = x % D;
    float o = lds[(0 * RH + r) * Dp + d];
#pragma unroll
    for (int w = 1; w < NW; ++w) o += lds[(w * RH + r) * Dp + d];
    const float gate = 1.f / (1.f + expf(-proj[(long)t * ld + gate_col + h0 + r]));
    stf<P>(out + (long)t * H * D + (long)(h0 + r) * D + d, o * gate);
  }
}

// ---- prompt attention on the matrix pipe (16-bit storage, D a multiple of 32).
// Workgroup = (16 consecutive positions of one sequence, one key/value group); its four waves take the group's query heads.
// Key list of the tile: pooled blocks 0 .. nb(last position) (padded to a multiple of 32), then the tokens from the first
// position's window start to the last position; a 32-key step is all pooled or all tokens.  Per step and head:
//   S^T = K Q^T as two 16-key MFMA tiles (A = 16 keys x 32 d straight from the cache rows, B = the queries);
//   P = visible ? sigmoid(S scale + bias) : 0 in fp32, lane (query j, key quad g) holding keys 4g .. 4g+3 of both tiles --
//   which IS the lane's share of the B operand of O^T += V^T P^T over the step's 32 keys when V^T's k index runs over
//   (tile 0: 4g..4g+3, tile 1: 4g..4g+3): no data moves between the two products;
//   V^T (A operand: 16 d x those 8 keys) is gathered from a [32 keys][D] copy of the value rows in LDS.
// Scores and weights stay fp32-exact on a bf16 / f16 matrix pipe by splitting the fp32 factor into a high and a low 16-bit
// half (x = hi + lo to 2^-17): q, the pooled means (held in fp32) and the weights go through two MFMAs instead of one.
template <typename P> __device__ __forceinline__ void split8(const float* v, u32x4& hi, u32x4& lo) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const u16 h0 = P::from_f(v[2 * e]), h1 = P::from_f(v[2 * e + 1]);
    const u16 l0 = P::from_f(v[2 * e] - P::to_f(h0)), l1 = P::from_f(v[2 * e + 1] - P::to_f(h1));
    hi[e] = (unsigned)h0 | ((unsigned)h1 << 16);
    lo[e] = (unsigned)l0 | ((unsigned)l1 << 16);
  }
}

template <typename P, int NS>
__global__ __launch_bounds__(256) void pwa_attend_mfma_kernel(u16* __restrict__ out, const float* __restrict__ q, UmbPagedKV kv,
                                                              const float* __restrict__ proj, int ld, int gate_col,
                                                              const u16* __restrict__ pos_bias, const int* __restrict__ seq_slot,
                                                              const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                              const int* __restrict__ seq_len, int H, int G, int window, int pool,
                                                              float scale) {
  constexpr int D = NS * 32, LD = D + 8;              // LDS row stride: 16 bytes of padding spread the key quads over the banks
  extern __shared__ __attribute__((aligned(16))) u16 vt_all[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g4 = lane >> 4;
  u16* v_hi = vt_all + (long)wave * (2 * 32 * LD + 32 * 4);   // [32][LD] values, [32][LD] low halves (pooled steps), [32] offsets
  u16* v_lo = v_hi + 32 * LD;
  long* offs = reinterpret_cast<long*>(v_lo + 32 * LD);
  const int b = blockIdx.y, g = blockIdx.z;
  const int n = seq_len[b], q0 = blockIdx.x * 16;
  if (q0 >= n) return;
  const int slot = seq_slot[b], row0 = seq_row0[b], pos0 = seq_pos0[b];
  const int nq = n - q0 < 16 ? n - q0 : 16;
  const int i_first = pos0 + q0, i_last = i_first + nq - 1;
  const bool q_ok = j < nq;
  const int i_j = i_first + (q_ok ? j : nq - 1);
  const long qrow = row0 + q0 + (q_ok ? j : nq - 1);
  const int nb_j = i_j - window + 1 >= pool ? (i_j - window + 1) / pool : 0;
  const int nb_max = i_last - window + 1 >= pool ? (i_last - window + 1) / pool : 0;
  const int j_lo = i_first - window + 1 > 0 ? i_first - window + 1 : 0;
  const int tok0 = (nb_max + 31) & ~31, total = tok0 + (i_last - j_lo + 1);
  const int R = H / G;
  for (int r = wave; r < R; r += 4) {
    const int h = g * R + r;
    u32x4 qhi[NS], qlo[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      float v[8];
      const f32x4 a = *reinterpret_cast<const f32x4*>(q + qrow * H * D + (long)h * D + 32 * s + 8 * g4);
      const f32x4 c = *reinterpret_cast<const f32x4*>(q + qrow * H * D + (long)h * D + 32 * s + 8 * g4 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = c[e]; }
      split8<P>(v, qhi[s], qlo[s]);
    }
    const float bias = pos_bias ? P::to_f(pos_bias[h]) : 0.f;
    f32x4 o[2 * NS];
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = 0; base < total; base += 32) {
      const bool pooled = base < tok0;
      // element offsets of the step's 32 keys (-1: no such key)
      if (lane < 32) {
        const int kx = base + lane;
        long off = -1;
        if (pooled) { if (kx < nb_max) off = pkv_blk(kv, slot, kx, pool, g, G, D); }
        else if (kx < total) off = pkv_tok(kv, slot, j_lo + (kx - tok0), g, G, D);
        offs[lane] = off;
      }
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
      // value rows -> LDS: 32 x D / 8 pieces of 8 features, NS pieces... (4 D / 64 = 2 NS per lane)
#pragma unroll
      for (int i = 0; i < 2 * NS; ++i) {
        const int p = lane + 64 * i, m = p / (D / 8), dp = (p % (D / 8)) * 8;
        const long off = offs[m];
        u32x4 hi = u32x4{0u, 0u, 0u, 0u}, lo = u32x4{0u, 0u, 0u, 0u};
        if (off >= 0) {
          if (pooled) {
            float v[8];
            const f32x4 a = *reinterpret_cast<const f32x4*>(kv.vp + off + dp);
            const f32x4 c = *reinterpret_cast<const f32x4*>(kv.vp + off + dp + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = c[e]; }
            split8<P>(v, hi, lo);
          } else {
            hi = *reinterpret_cast<const u32x4*>(reinterpret_cast<const u16*>(kv.v) + off + dp);
          }
        }
        *reinterpret_cast<u32x4*>(v_hi + m * LD + dp) = hi;
        if (pooled) *reinterpret_cast<u32x4*>(v_lo + m * LD + dp) = lo;
      }
      // scores of the two 16-key tiles
      f32x4 sc[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        const long off = offs[16 * u + j];
        const long offc = off >= 0 ? off : 0;
        if (pooled) {
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            float v[8];
            const f32x4 a = *reinterpret_cast<const f32x4*>(kv.kp + offc + 32 * s + 8 * g4);
            const f32x4 c = *reinterpret_cast<const f32x4*>(kv.kp + offc + 32 * s + 8 * g4 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = c[e]; }
            u32x4 khi, klo;
            split8<P>(v, khi, klo);
            sc[u] = P::mfma(khi, qhi[s], sc[u]);
            sc[u] = P::mfma(khi, qlo[s], sc[u]);
            sc[u] = P::mfma(klo, qhi[s], sc[u]);
          }
        } else {
          u32x4 kf[NS];
#pragma unroll
          for (int s = 0; s < NS; ++s)
            kf[s] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const u16*>(kv.k) + offc + 32 * s + 8 * g4);
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            sc[u] = P::mfma(kf[s], qhi[s], sc[u]);
            sc[u] = P::mfma(kf[s], qlo[s], sc[u]);
          }
        }
      }
      // weights: lane (query j, quad g4) holds keys 16 u + 4 g4 + r of the step
      float w[8];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int kk = base + 16 * u + 4 * g4 + rr;
          bool vis;
          if (pooled) vis = kk < nb_j;
          else { const int jt = j_lo + (kk - tok0); vis = jt <= i_j && jt > i_j - window; }
          w[4 * u + rr] = (vis && q_ok) ? 1.f / (1.f + expf(-(sc[u][rr] * scale + bias))) : 0.f;
        }
      u32x4 phi, plo;
      split8<P>(w, phi, plo);
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
      // O^T[d][query] += V^T[d][keys] P^T[keys][query]: lane (d row j of tile dt, quad g4) gathers its 8 keys' values
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) {
        unsigned e[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) e[m] = v_hi[((m >> 2) * 16 + 4 * g4 + (m & 3)) * LD + 16 * dt + j];
        const u32x4 va = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
        o[dt] = P::mfma(va, phi, o[dt]);
        o[dt] = P::mfma(va, plo, o[dt]);
        if (pooled) {
#pragma unroll
          for (int m = 0; m < 8; ++m) e[m] = v_lo[((m >> 2) * 16 + 4 * g4 + (m & 3)) * LD + 16 * dt + j];
          const u32x4 vl = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
          o[dt] = P::mfma(vl, phi, o[dt]);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    // lane holds O^T[d = 16 dt + 4 g4 + rr][query j]
    if (q_ok) {
      const float gate = 1.f / (1.f + expf(-proj[qrow * ld + gate_col + h]));
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) {
        u32x2 pk;
        pk[0] = pack2<P>(o[dt][0] * gate, o[dt][1] * gate);
        pk[1] = pack2<P>(o[dt][2] * gate, o[dt][3] * gate);
        *reinterpret_cast<u32x2*>(out + qrow * H * D + (long)h * D + 16 * dt + 4 * g4) = pk;
      }
    }
  }
}

static inline bool pkv_ok(const UmbPagedKV* kv) {
  return kv && kv->k && kv->v && kv->kp && kv->vp && kv->pages && kv->page >= 1 && kv->max_pages >= 1;
}

extern "C" int umb_pwa_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const int* pos, const int* slot,
                            const float* freq, int T, int H, int G, int D, int rot_dims, float eps, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || D < 1 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) || !q || !pkv_ok(kv) || !proj || !pos ||
      !slot || (rot_dims && !freq))
    return UMB_EINVAL;
  const long n = (long)T * (H + G);
  DISPATCH_SEQ_DTYPE(dtype, {
    hipLaunchKernelGGL(pwa_prep_kernel<P>, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, st, q, *kv, proj, ld, pos, slot, freq, T, H,
                       G, D, rot_dims, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_pwa_pool(const UmbPagedKV* kv, const int* seq_slot, const int* seq_pos0, const int* seq_len, int B, int max_len,
                            int G, int D, int pool, int dtype, hipStream_t st) {
  if (B < 1 || max_len < 1 || G < 1 || D < 1 || pool < 1 || !pkv_ok(kv) || !seq_slot || !seq_pos0 || !seq_len) return UMB_EINVAL;
  const int nb = max_len / pool + 1;             // at most this many blocks end inside max_len consecutive positions
  DISPATCH_SEQ_DTYPE(dtype, {
    hipLaunchKernelGGL(pwa_pool_kernel<P>, dim3(nb, B, G), dim3(64), 0, st, *kv, seq_slot, seq_pos0, seq_len, G, D, pool);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_pwa_attend(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                              const void* pos_bias, const int* pos, const int* slot, int T, int H, int G, int D, int window,
                              int pool, float scale, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || D > 64 * PWA_MAXC || window < 1 || pool < 1 || !out || !q || !pkv_ok(kv) ||
      !proj || !pos || !slot)
    return UMB_EINVAL;
  const int R = H / G;
  const int rh = R % 8 == 0 ? 8 : (R % 4 == 0 ? 4 : (R % 2 == 0 ? 2 : 1));     // heads of one group per workgroup
  const int Dp = (D + 3) & ~3;
  const dim3 grid(T, H / rh);
  // few workgroups (decoding): sixteen waves share a query's keys, so a step's latency is one or two rounds; many (prompts):
  // four, the chip is full anyway.  The choice changes the order in which a query's partial sums are added, nothing else.
  int nw = (long)T * (H / rh) < 1024 ? 16 : 4;
  if (nw == 16 && ((size_t)16 * rh * Dp + 16 * (rh * 64 + 128)) * sizeof(float) > 96 * 1024) nw = 4;     // LDS of one CU
  const size_t lds = ((size_t)nw * rh * Dp + nw * (rh * 64 + 128)) * sizeof(float);
#define PWA_LAUNCH(RH, NC, NW)                                                                                            \
  do {                                                                                                                    \
    if (ensure_dynamic_lds<pwa_attend_kernel<P, RH, NC, NW>>(lds) != UMB_OK) return UMB_EHIP;                             \
    hipLaunchKernelGGL((pwa_attend_kernel<P, RH, NC, NW>), grid, dim3(NW * 64), lds, st, (E*)out, q, *kv, proj, ld,       \
                       gate_col, (const E*)pos_bias, pos, slot, T, H, G, D, window, pool, scale);                         \
  } while (0)
#define PWA_NC(RH, NW)                                                                                                    \
  if (D <= 64) PWA_LAUNCH(RH, 1, NW); else if (D <= 128) PWA_LAUNCH(RH, 2, NW); else PWA_LAUNCH(RH, 4, NW)
#define PWA_CASE(RH)                                                                                                       \
  case RH:                                                                                                                 \
    if (nw == 16) { PWA_NC(RH, 16); } else { PWA_NC(RH, 4); }                                                              \
    break;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    switch (rh) { PWA_CASE(8) PWA_CASE(4) PWA_CASE(2) default: PWA_CASE(1) }
  })
#undef PWA_CASE
#undef PWA_NC
#undef PWA_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_pwa_attend_tiled(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                                    const void* pos_bias, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                                    const int* seq_len, int B, int max_len, int H, int G, int D, int window, int pool, float scale,
                                    int dtype, hipStream_t st) {
  if (B < 1 || max_len < 1 || H < 1 || G < 1 || H % G || D < 32 || D > 256 || D % 32 || window < 1 || pool < 1 || !out || !q ||
      !pkv_ok(kv) || !proj || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len || dtype == UMB_SEQ_F32)
    return UMB_EINVAL;
  const dim3 grid((max_len + 15) / 16, B, G);
  const size_t lds = 4 * (size_t)(2 * 32 * (D + 8) + 128) * sizeof(u16);
#define PWA_MFMA_CASE(NS)                                                                                                  \
  case NS:                                                                                                                 \
    if (ensure_dynamic_lds<pwa_attend_mfma_kernel<P, NS>>(lds) != UMB_OK) return UMB_EHIP;                                 \
    hipLaunchKernelGGL((pwa_attend_mfma_kernel<P, NS>), grid, dim3(256), lds, st, (u16*)out, q, *kv, proj, ld, gate_col,   \
                       (const u16*)pos_bias, seq_slot, seq_row0, seq_pos0, seq_len, H, G, window, pool, scale);            \
    break;
  if (dtype == UMB_SEQ_BF16) {
    using P = BF16;
    switch (D / 32) { PWA_MFMA_CASE(1) PWA_MFMA_CASE(2) PWA_MFMA_CASE(3) PWA_MFMA_CASE(4) PWA_MFMA_CASE(5) PWA_MFMA_CASE(6)
                      PWA_MFMA_CASE(7) PWA_MFMA_CASE(8) default: return UMB_EINVAL; }
  } else if (dtype == UMB_SEQ_F16) {
    using P = F16;
    switch (D / 32) { PWA_MFMA_CASE(1) PWA_MFMA_CASE(2) PWA_MFMA_CASE(3) PWA_MFMA_CASE(4) PWA_MFMA_CASE(5) PWA_MFMA_CASE(6)
                      PWA_MFMA_CASE(7) PWA_MFMA_CASE(8) default: return UMB_EINVAL; }
  } else {
    return UMB_EINVAL;
  }
#undef PWA_MFMA_CASE
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
