// Latent attention over a paged store: queries and keys/values pass through low-rank latents, and the cache holds per token
// only the normed key/value latent c [kv_rank] and one rotated key part k_rot [rot_dim] that every head shares -- one row of
// Dk = kv_rank + rot_dim elements.
//
// The per-head keys W_uk[h] c and values W_uv[h] c are never formed.  With q = [q_nope | q_rot] per head,
//     q_nope . (W_uk[h] c_j) = (W_uk[h]^T q_nope) . c_j            -> the query is carried into the latent space once,
//     sum_j p_j (W_uv[h] c_j) = W_uv[h] (sum_j p_j c_j)            -> the value up-projection is applied once, after the sum,
// so attention runs as H query heads against ONE shared key/value row per token: score = (qa . [c | k_rot]) * scale with
// qa = [W_uk^T q_nope | rope(q_rot)], and the weighted sum is taken over c.  A decode step reads each cached row once for
// all heads; a prompt tile re-uses a staged row for 16 positions x H heads.
//
// Visibility: position i sees j with 0 <= i - j < window.  Softmax with a sink: the denominator also holds exp(sink[h]),
// which has no key and no value and is not scaled.  Scores, weights, maxima and sums are fp32; rotary angles are
// pos * freq[i] in fp32 through the full-range sincosf; pairs (2i, 2i+1) of the first rot_dims features of the rotated part
// turn, the rest pass.
#include "seq_common.h"

static inline bool lat_kv_ok(const UmbPagedKV* kv) { return kv && kv->k && kv->pages && kv->page >= 1 && kv->max_pages >= 1; }

// ---- norms of the two latents, rotation of the shared key part, cache append.  One wave per (token, part): part 0 = the
// query latent, part 1 = the key/value latent + rotated key.
template <typename P>
__global__ __launch_bounds__(256) void lat_prep_kernel(typename El<P>::type* __restrict__ cq, UmbPagedKV kv,
                                                       const float* __restrict__ proj, int ld,
                                                       const typename El<P>::type* __restrict__ w_q,
                                                       const typename El<P>::type* __restrict__ w_kv, const int* __restrict__ pos,
                                                       const int* __restrict__ slot, const float* __restrict__ freq, int T,
                                                       int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps) {
  typedef typename El<P>::type E;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long id = (long)blockIdx.x * 4 + wave;
  if (id >= 2L * T) return;
  const int t = (int)(id >> 1), part = (int)(id & 1);
  const float* src = proj + (long)t * ld + (part ? q_rank : 0);
  const int n = part ? kv_rank : q_rank;
  float ss = 0.f;
  for (int i = lane; i < n; i += 64) { const float v = src[i]; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)n + eps);
  if (!part) {
    for (int i = lane; i < n; i += 64) stf<P>(cq + (long)t * q_rank + i, src[i] * f * ldf<P>(w_q + i));
    return;
  }
  const int p = pos[t];
  E* row = reinterpret_cast<E*>(kv.k) + pkv_tok(kv, slot[t], p, 0, 1, kv_rank + rot_dim);
  for (int i = lane; i < n; i += 64) stf<P>(row + i, src[i] * f * ldf<P>(w_kv + i));
  const float* kr = src + kv_rank;
  const float pf = (float)p;
  for (int m = lane; m < (rot_dim + 1) / 2; m += 64) {
    const int d0 = 2 * m, d1 = 2 * m + 1;
    float u = kr[d0], v = d1 < rot_dim ? kr[d1] : 0.f;
    if (d1 < rot_dims) {
      float sn, cs;
      sincosf(pf * freq[m], &sn, &cs);
      const float ru = u * cs - v * sn, rv = v * cs + u * sn;
      u = ru; v = rv;
    }
    stf<P>(row + kv_rank + d0, u);
    if (d1 < rot_dim) stf<P>(row + kv_rank + d1, v);
  }
}

// ---- queries: unrotated parts to the storage dtype (they feed the product with W_uk^T), rotated parts turned in fp32
template <typename P>
__global__ __launch_bounds__(256) void lat_qsplit_kernel(typename El<P>::type* __restrict__ qn, float* __restrict__ qa,
                                                         const float* __restrict__ q, const int* __restrict__ pos,
                                                         const float* __restrict__ freq, int T, int H, int D, int R, int kv_rank,
                                                         int rot_dims) {
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  const int per = D + (R + 1) / 2;                      // work items of one (token, head): D copies + R / 2 pairs
  if (id >= (long)T * H * per) return;
  const int e = (int)(id % per);
  const long th = id / per;
  const int t = (int)(th / H);
  const float* src = q + th * (D + R);
  if (e < D) { stf<P>(qn + th * D + e, src[e]); return; }
  const int m = e - D, d0 = 2 * m, d1 = 2 * m + 1;
  float u = src[D + d0], v = d1 < R ? src[D + d1] : 0.f;
  if (d1 < rot_dims) {
    float sn, cs;
    sincosf((float)pos[t] * freq[m], &sn, &cs);
    const float ru = u * cs - v * sn, rv = v * cs + u * sn;
    u = ru; v = rv;
  }
  float* dst = qa + th * (kv_rank + R) + kv_rank;
  dst[d0] = u;
  if (d1 < R) dst[d1] = v;
}

// ---- attention, one workgroup per (token, RH heads).  The NW waves take the 64-key rounds w, w + NW, ... of the window's keys
// in position order; inside a round lane = key for the scores (the key's row against the queries in LDS), then lane = value
// column for the weighted sum, the round's weights broadcast one key at a time.  Each wave keeps a running maximum and
// denominator per head (the usual rescaling when the maximum grows); the waves' partial results are merged through LDS in
// wave order together with the sink.  Which keys land in which wave and round depends on the query's position alone -- never
// on the batch or on how the prompt was cut.
constexpr int LAT_MAXC = 8;      // value columns per lane: kv_rank <= 512

template <typename P, int RH, int NC, int NW>
__global__ __launch_bounds__(NW * 64) void lat_attend_kernel(typename El<P>::type* __restrict__ out, const float* __restrict__ qa,
                                                             UmbPagedKV kv, const typename El<P>::type* __restrict__ sink,
                                                             const int* __restrict__ pos, const int* __restrict__ slot_, int T,
                                                             int H, int Dc, int R, int window, float scale) {
  typedef typename El<P>::type E;
  extern __shared__ float lds[];
  constexpr int KB = 8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Dk = Dc + R, Dp = (Dk + 3) & ~3;
  // [RH][Dp] queries (later [NW][RH][Dp] partial sums), [NW][2 RH] maxima and denominators, per wave [RH][64] weights + offsets
  float* q_s = lds;
  float* ml_s = lds + NW * RH * Dp;
  float* w_s = ml_s + NW * 2 * RH + wave * (RH * 64 + 128);
  long* off_s = reinterpret_cast<long*>(w_s + RH * 64);
  const int t = blockIdx.x, h0 = blockIdx.y * RH;
  const int i = pos[t], slot = slot_[t];
  for (int x = threadIdx.x; x < RH * Dk; x += NW * 64) {
    const int r = x / Dk, d = x % Dk;
    q_s[r * Dp + d] = h0 + r < H ? qa[((long)t * H + h0 + r) * Dk + d] : 0.f;
  }
  __syncthreads();
  const int j_lo = i - window + 1 > 0 ? i - window + 1 : 0;
  const int n_keys = i - j_lo + 1;
  const bool vec = (Dk & 7) == 0 && sizeof(E) == 2;
  float acc[RH][NC], m_run[RH], l_run[RH];
#pragma unroll
  for (int r = 0; r < RH; ++r) {
    m_run[r] = -INFINITY;
    l_run[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[r][c] = 0.f;
  }
  int dcl[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) dcl[c] = lane + 64 * c < Dc ? lane + 64 * c : Dc - 1;
  for (int base = wave * 64; base < n_keys; base += NW * 64) {
    const int kx = base + lane;
    float s[RH];
#pragma unroll
    for (int r = 0; r < RH; ++r) s[r] = 0.f;
    long off = 0;
    if (kx < n_keys) {
      off = pkv_tok(kv, slot, j_lo + kx, 0, 1, Dk);
      const E* kr = reinterpret_cast<const E*>(kv.k) + off;
      bool done = false;
      if constexpr (sizeof(E) == 2) {
        if (vec) {
          for (int d = 0; d < Dk; d += 64) {            // eight 16-byte loads in flight, then their 64 x RH products
            u32x4 kk[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) kk[u] = *reinterpret_cast<const u32x4*>(kr + (d + 8 * u < Dk ? d + 8 * u : 0));
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              if (d + 8 * u >= Dk) break;
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
        for (int d = 0; d < Dk; ++d) {
          const float kd = ldf<P>(kr + d);
#pragma unroll
          for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + d] * kd;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RH; ++r) {
      const float sv = kx < n_keys ? s[r] * scale : -INFINITY;
      const float m_new = fmaxf(m_run[r], wave_max(sv));          // finite: every round has at least one key
      const float fac = expf(m_run[r] - m_new);                   // 0 on the first round (m_run = -inf)
      const float pw = kx < n_keys ? expf(sv - m_new) : 0.f;
      l_run[r] = l_run[r] * fac + wave_sum(pw);
      m_run[r] = m_new;
#pragma unroll
      for (int c = 0; c < NC; ++c) acc[r][c] *= fac;
      w_s[r * 64 + lane] = pw;
    }
    off_s[lane] = off;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int cnt = n_keys - base < 64 ? n_keys - base : 64;
    for (int j0 = 0; j0 < cnt; j0 += KB) {
      float vv[KB][NC];
#pragma unroll
      for (int u = 0; u < KB; ++u) {
        const long oj = off_s[j0 + u < cnt ? j0 + u : cnt - 1];
#pragma unroll
        for (int c = 0; c < NC; ++c) vv[u][c] = ldf<P>(reinterpret_cast<const E*>(kv.k) + oj + dcl[c]);
      }
#pragma unroll
      for (int u = 0; u < KB; ++u) {
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
  for (int r = 0; r < RH; ++r) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < Dc) lds[(wave * RH + r) * Dp + d] = acc[r][c];
    }
    if (lane == 0) { ml_s[(wave * RH + r) * 2] = m_run[r]; ml_s[(wave * RH + r) * 2 + 1] = l_run[r]; }
  }
  __syncthreads();
  for (int x = threadIdx.x; x < RH * Dc; x += NW * 64) {
    const int r = x / Dc, d = x % Dc;
    if (h0 + r >= H) continue;
    const float sk = sink ? ldf<P>(sink + h0 + r) : -INFINITY;
    float M = sk;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, ml_s[(w * RH + r) * 2]);
    float o = 0.f, L = sink ? expf(sk - M) : 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = ml_s[(w * RH + r) * 2];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      o += lds[(w * RH + r) * Dp + d] * f;
      L += ml_s[(w * RH + r) * 2 + 1] * f;
    }
    stf<P>(out + ((long)t * H + h0 + r) * Dc + d, o / L);
  }
}

extern "C" int umb_lat_prep(void* cq, const UmbPagedKV* kv, const float* proj, int ld, const void* w_q, const void* w_kv,
                            const int* pos, const int* slot, const float* freq, int T, int q_rank, int kv_rank, int rot_dim,
                            int rot_dims, float eps, int dtype, hipStream_t st) {
  if (T < 1 || q_rank < 1 || kv_rank < 1 || rot_dim < 0 || rot_dims < 0 || rot_dims > rot_dim || (rot_dims & 1) || !cq ||
      !lat_kv_ok(kv) || !proj || !w_q || !w_kv || !pos || !slot || (rot_dims && !freq) || ld < q_rank + kv_rank + rot_dim)
    return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(lat_prep_kernel<P>, dim3((unsigned)((2L * T + 3) / 4)), dim3(256), 0, st, (E*)cq, *kv, proj, ld,
                       (const E*)w_q, (const E*)w_kv, pos, slot, freq, T, q_rank, kv_rank, rot_dim, rot_dims, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_lat_qsplit(void* qn, float* qa, const float* q, const int* pos, const float* freq, int T, int H, int D, int R,
                              int kv_rank, int rot_dims, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || D < 1 || R < 0 || kv_rank < 1 || rot_dims < 0 || rot_dims > R || (rot_dims & 1) || !qn || !qa || !q ||
      !pos || (rot_dims && !freq))
    return UMB_EINVAL;
  const long n = (long)T * H * (D + (R + 1) / 2);
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(lat_qsplit_kernel<P>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (E*)qn, qa, q, pos, freq, T, H,
                       D, R, kv_rank, rot_dims);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_lat_attend(void* out, const float* qa, const UmbPagedKV* kv, const void* sink, const int* pos, const int* slot,
                              int T, int H, int kv_rank, int rot_dim, int window, float scale, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || kv_rank < 1 || kv_rank > 64 * LAT_MAXC || rot_dim < 0 || window < 1 || !out || !qa || !lat_kv_ok(kv) ||
      !pos || !slot)
    return UMB_EINVAL;
  const int Dk = kv_rank + rot_dim, Dp = (Dk + 3) & ~3;
  // heads of one workgroup: all of them share the keys, so as many as the register budget of the partial sums allows
  const int nc = (kv_rank + 63) / 64;
  int rh = nc <= 2 ? 8 : (nc <= 4 ? 4 : 2);
  while (rh > 1 && rh / 2 >= H) rh >>= 1;
  const int hb = (H + rh - 1) / rh;
  const dim3 grid(T, hb);
  int nw = (long)T * hb < 1024 ? 16 : 4;
  auto lds_of = [&](int w) { return ((size_t)w * rh * Dp + (size_t)w * 2 * rh + (size_t)w * (rh * 64 + 128)) * sizeof(float); };
  if (nw == 16 && lds_of(16) > 128 * 1024) nw = 4;
  if (lds_of(nw) > 160 * 1024) return UMB_EINVAL;
  const size_t lds = lds_of(nw);
#define LAT_LAUNCH(RH, NC, NW)                                                                                            \
  do {                                                                                                                    \
    if (ensure_dynamic_lds<lat_attend_kernel<P, RH, NC, NW>>(lds) != UMB_OK) return UMB_EHIP;                             \
    hipLaunchKernelGGL((lat_attend_kernel<P, RH, NC, NW>), grid, dim3(NW * 64), lds, st, (E*)out, qa, *kv, (const E*)sink, \
                       pos, slot, T, H, kv_rank, rot_dim, window, scale);                                                 \
  } while (0)
#define LAT_NW(RH, NC)                                                                                                    \
  if (nw == 16) LAT_LAUNCH(RH, NC, 16); else LAT_LAUNCH(RH, NC, 4)
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    if (nc <= 1) { if (rh == 8) { LAT_NW(8, 1); } else if (rh == 4) { LAT_NW(4, 1); } else if (rh == 2) { LAT_NW(2, 1); } else { LAT_NW(1, 1); } }
    else if (nc <= 2) { if (rh == 8) { LAT_NW(8, 2); } else if (rh == 4) { LAT_NW(4, 2); } else if (rh == 2) { LAT_NW(2, 2); } else { LAT_NW(1, 2); } }
    else if (nc <= 4) { if (rh == 4) { LAT_NW(4, 4); } else if (rh == 2) { LAT_NW(2, 4); } else { LAT_NW(1, 4); } }
    else { if (rh == 2) { LAT_NW(2, 8); } else { LAT_NW(1, 8); } }
  })
#undef LAT_NW
#undef LAT_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_lat_attend_tiled_ok(int H, int kv_rank, int rot_dim, int dtype) {
  (void)H; (void)kv_rank; (void)rot_dim; (void)dtype;
  return 0;
}

extern "C" int umb_lat_attend_tiled(void* out, const float* qa, const UmbPagedKV* kv, const void* sink, const int* seq_slot,
                                    const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int max_len, int H,
                                    int kv_rank, int rot_dim, int window, float scale, int dtype, hipStream_t st) {
  (void)out; (void)qa; (void)kv; (void)sink; (void)seq_slot; (void)seq_row0; (void)seq_pos0; (void)seq_len; (void)B;
  (void)max_len; (void)H; (void)kv_rank; (void)rot_dim; (void)window; (void)scale; (void)dtype; (void)st;
  return UMB_EINVAL;
}
