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
#include <cstdlib>

constexpr float LOG2E = 1.4426950408889634f;

static inline bool lat_kv_ok(const UmbPagedKV* kv) { return kv && kv->k && kv->pages && kv->page >= 1 && kv->max_pages >= 1; }

// ---- norms of the two latents, rotation of the shared key part, cache append.  One workgroup per (token, part): part 0 =
// the query latent, part 1 = the key/value latent + rotated key.
template <typename P>
__global__ __launch_bounds__(256) void lat_prep_kernel(typename El<P>::type* __restrict__ cq, UmbPagedKV kv,
                                                       const float* __restrict__ proj, int ld,
                                                       const typename El<P>::type* __restrict__ w_q,
                                                       const typename El<P>::type* __restrict__ w_kv, const int* __restrict__ pos,
                                                       const int* __restrict__ slot, const float* __restrict__ freq, int T,
                                                       int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps) {
  typedef typename El<P>::type E;
  __shared__ float red[8];
  const int lane = threadIdx.x;
  const int t = blockIdx.x >> 1, part = blockIdx.x & 1;
  const float* src = proj + (long)t * ld + (part ? q_rank : 0);
  const int n = part ? kv_rank : q_rank;
  float ss = 0.f;
#pragma unroll 4
  for (int i = lane; i < n; i += 256) { const float v = src[i]; ss += v * v; }
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)n + eps);
  if (!part) {
    for (int i = lane; i < n; i += 256) stf<P>(cq + (long)t * q_rank + i, src[i] * f * ldf<P>(w_q + i));
    return;
  }
  const int p = pos[t];
  E* row = reinterpret_cast<E*>(kv.k) + pkv_tok(kv, slot[t], p, 0, 1, kv_rank + rot_dim);
  for (int i = lane; i < n; i += 256) stf<P>(row + i, src[i] * f * ldf<P>(w_kv + i));
  const float* kr = src + kv_rank;
  const float pf = (float)p;
  for (int m = lane; m < (rot_dim + 1) / 2; m += 256) {
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
constexpr int LAT_MAXC = 16;     // value columns per lane: kv_rank <= 1024

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

// ---- prompt attention on the matrix pipe (16-bit storage; Dk a multiple of 8, kv_rank a multiple of 16).
// Workgroup = (16 consecutive positions of one sequence, a block of 4 HPW heads); wave w owns HPW heads.  The tile's keys -- from
// the first position's window start to the last position -- are walked in steps of 32 by the whole workgroup: the step's 32
// cached rows (all Dk features) are staged ONCE into a shared LDS tile and serve every head of the workgroup, as keys and as
// values; the next step's rows are already in flight (in registers) while the current one is used, so the one global round
// trip of a step hides behind its matrix products, and the small tile leaves room for several workgroups per CU.
// Per step and head:
//   S^T = K Q^T as two 16-key MFMA tiles (A = 16 keys x 32 features read from the LDS tile, B = the queries, rounded to the
//         storage dtype once, when the tile starts);
//   online softmax in fp32: lane (query j, key quad g) holds keys 4g .. 4g+3 of both tiles; the row maximum and sum are
//         finished over the four lanes of a query by two shuffles; accumulators are rescaled when the maximum grows;
//   O^T += V^T P^T: the lane's eight weights ARE its share of the B operand when V^T's k index runs over (tile 0: 4g .. 4g+3,
//         tile 1: 4g .. 4g+3); V^T (A: 16 features x those 8 keys) is gathered from the LDS tile.
// The sink joins the denominator at the end.  NSM / NVM bound the unrolled register arrays (key steps of 32 features, value
// tiles of 16 features); the actual counts are run-time.
template <typename P, int NSM, int NVM, int HPW>
__global__ __launch_bounds__(256) void lat_attend_mfma_kernel(u16* __restrict__ out, const float* __restrict__ qa, UmbPagedKV kv,
                                                              const u16* __restrict__ sink, const int* __restrict__ seq_slot,
                                                              const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                              const int* __restrict__ seq_len, int H, int Dc, int R, int window,
                                                              float scale) {
  extern __shared__ __attribute__((aligned(16))) u16 lat_lds[];
  constexpr int NLD = (NSM + 1) / 2;                  // 16-byte chunks of a row per staging thread: Dk / 8 chunks over 8 threads
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g4 = lane >> 4;
  const int Dk = Dc + R, LD = Dk + 8;                 // LDS row stride: 16 bytes of padding spread the key quads over the banks
  const int ns = (Dk + 31) >> 5, nv = Dc >> 4, nch = Dk >> 3;
  constexpr int LT = 36;                              // row stride of the transposed tile: 32 keys + 8 bytes of padding
  u16* v_s = lat_lds;                                 // [32][LD]: the step's rows as cached (keys: A operand of S^T = K Q^T)
  u16* v_t = lat_lds + 32 * LD;                       // [Dc][LT]: their first Dc features transposed (values: A operand of O^T)
  const int b = blockIdx.y;
  const int n = seq_len[b], q0 = blockIdx.x * 16;
  if (q0 >= n) return;                                // the whole workgroup
  const int h0 = (blockIdx.z * 4 + wave) * HPW;
  const bool active = h0 < H;                         // a wave without heads still stages rows and meets the barriers
  const int slot = seq_slot[b], row0 = seq_row0[b], pos0 = seq_pos0[b];
  const int nq = n - q0 < 16 ? n - q0 : 16;
  const int i_first = pos0 + q0, i_last = i_first + nq - 1;
  const bool q_ok = j < nq;
  const int i_j = i_first + (q_ok ? j : nq - 1);
  const long qrow = row0 + q0 + (q_ok ? j : nq - 1);
  const int j_lo = i_first - window + 1 > 0 ? i_first - window + 1 : 0;
  const int total = i_last - j_lo + 1;
  const float scale2 = scale * LOG2E;
  const u16* kbase = reinterpret_cast<const u16*>(kv.k);
  u32x4 qf[HPW][NSM];
  f32x4 o[HPW][NVM];
  float m_run[HPW], l_run[HPW];
  bool h_ok[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    h_ok[hh] = h0 + hh < H;
    const float* qr = qa + (qrow * H + (h_ok[hh] ? h0 + hh : H - 1)) * Dk;
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      const int d = 32 * s + 8 * g4;
      qf[hh][s] = u32x4{0u, 0u, 0u, 0u};
      if (s < ns && d < Dk) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(qr + d), c = *reinterpret_cast<const f32x4*>(qr + d + 4);
        qf[hh][s] = u32x4{pack2<P>(a[0], a[1]), pack2<P>(a[2], a[3]), pack2<P>(c[0], c[1]), pack2<P>(c[2], c[3])};
      }
    }
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) o[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
  }
  // staging role of a thread: key row sm of the step, 16-byte chunks sc, sc + 8, ... of that row
  const int sm = threadIdx.x & 31, sc = threadIdx.x >> 5;
  u32x4 stage[NLD];
  auto fetch = [&](int base) {
    const int kx = base + sm;
    const long off = kx < total ? pkv_tok(kv, slot, j_lo + kx, 0, 1, Dk) : -1;
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      const int ch = sc + 8 * u;
      stage[u] = (off >= 0 && ch < nch) ? *reinterpret_cast<const u32x4*>(kbase + off + 8 * ch) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  fetch(0);
  for (int base = 0; base < total; base += 32) {
    __syncthreads();                                  // every wave is done with the previous tile
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      const int ch = sc + 8 * u;
      if (ch < nch) {
        *reinterpret_cast<u32x4*>(v_s + sm * LD + 8 * ch) = stage[u];
        if (8 * ch < Dc) {                            // Dc is a multiple of 16: a chunk is all values or all rotated key part
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v_t[(8 * ch + 2 * e) * LT + sm] = (u16)(stage[u][e] & 0xffffu);
            v_t[(8 * ch + 2 * e + 1) * LT + sm] = (u16)(stage[u][e] >> 16);
          }
        }
      }
    }
    __syncthreads();
    if (base + 32 < total) fetch(base + 32);          // in flight while this step is used
    if (!active) continue;
    f32x4 sc2[HPW][2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) sc2[hh][u] = f32x4{0.f, 0.f, 0.f, 0.f};
      const u16* kr = v_s + (16 * u + j) * LD;
#pragma unroll
      for (int s = 0; s < NSM; ++s) {
        const int d = 32 * s + 8 * g4;
        if (s < ns) {
          const u32x4 kf = d < Dk ? *reinterpret_cast<const u32x4*>(kr + d) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) sc2[hh][u] = P::mfma(kf, qf[hh][s], sc2[hh][u]);
        }
      }
    }
    // which of the lane's eight keys this query sees: the same for every head
    bool vis[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int jt = j_lo + base + 16 * (e >> 2) + 4 * g4 + (e & 3);
      vis[e] = q_ok && jt <= i_j && jt > i_j - window;
    }
    u32x4 pf[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      // maxima and exponents in base 2 (scale2 = scale log2 e): one v_exp_f32 per weight
      float sv[8], mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sv[e] = vis[e] ? sc2[hh][e >> 2][e & 3] * scale2 : -INFINITY;
        mx = fmaxf(mx, sv[e]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[hh], mx);
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;          // a row that has seen no key yet: all weights 0
      const float fac = __builtin_amdgcn_exp2f(m_run[hh] - m_ref);
      float w[8], sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        w[e] = __builtin_amdgcn_exp2f(sv[e] - m_ref);
        sum += w[e];
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l_run[hh] = l_run[hh] * fac + sum;
      m_run[hh] = m_new;
      if (__ballot(fac != 1.f)) {                                    // the maximum moved for some row of the tile
#pragma unroll
        for (int dt = 0; dt < NVM; ++dt) {
          if (dt < nv) { o[hh][dt][0] *= fac; o[hh][dt][1] *= fac; o[hh][dt][2] *= fac; o[hh][dt][3] *= fac; }
        }
      }
      pf[hh] = u32x4{pack2<P>(w[0], w[1]), pack2<P>(w[2], w[3]), pack2<P>(w[4], w[5]), pack2<P>(w[6], w[7])};
    }
    // O^T[d][query] += V^T[d][keys] P^T[keys][query]: lane (d row j of tile dt, quad g4) reads its 8 keys' values
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) {
      if (dt < nv) {
        const u16* vr = v_t + (16 * dt + j) * LT + 4 * g4;
        const u32x2 t0 = *reinterpret_cast<const u32x2*>(vr), t1 = *reinterpret_cast<const u32x2*>(vr + 16);
        const u32x4 va = u32x4{t0[0], t0[1], t1[0], t1[1]};
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) o[hh][dt] = P::mfma(va, pf[hh], o[hh][dt]);
      }
    }
  }
  // lane holds O^T[d = 16 dt + 4 g4 + rr][query j]
  if (q_ok && active) {
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      if (!h_ok[hh]) continue;
      const float sk = sink ? P::to_f(sink[h0 + hh]) * LOG2E : -INFINITY;      // the running maximum is in base 2
      const float M = fmaxf(m_run[hh], sk);
      const float f = exp2f(m_run[hh] - M);
      const float inv = f / (l_run[hh] * f + (sink ? exp2f(sk - M) : 0.f));
#pragma unroll
      for (int dt = 0; dt < NVM; ++dt) {
        if (dt < nv) {
          u32x2 pk;
          pk[0] = pack2<P>(o[hh][dt][0] * inv, o[hh][dt][1] * inv);
          pk[1] = pack2<P>(o[hh][dt][2] * inv, o[hh][dt][3] * inv);
          *reinterpret_cast<u32x2*>(out + (qrow * H + h0 + hh) * Dc + 16 * dt + 4 * g4) = pk;
        }
      }
    }
  }
}

// ---- single tokens on the matrix pipe (16-bit storage): the 16 rows of the query tile are 16 HEADS of one token -- they
// all read the same cached rows, so one key fragment and one staged value tile serve sixteen heads.  Workgroup = (token,
// block of 16 heads); its four waves take the 32-key steps w, w + 4, ... of the window (which step lands in which wave depends
// on the token's position alone) with the same step body as the prompt kernel, then merge their running maxima, sums and
// partial outputs through LDS in wave order, where the sink joins the denominator.
template <typename P, int NSM, int NVM>
__global__ __launch_bounds__(256) void lat_decode_mfma_kernel(u16* __restrict__ out, const float* __restrict__ qa, UmbPagedKV kv,
                                                              const u16* __restrict__ sink, const int* __restrict__ pos,
                                                              const int* __restrict__ slot_, int H, int Dc, int R, int window,
                                                              float scale) {
  extern __shared__ __attribute__((aligned(16))) u16 lat_lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g4 = lane >> 4;
  const int Dk = Dc + R, LD = Dc + 8;
  const int ns = (Dk + 31) >> 5, nv = Dc >> 4;
  u16* v_s = lat_lds + (long)wave * (32 * LD + 32 * 4);
  long* offs = reinterpret_cast<long*>(v_s + 32 * LD);
  const int t = blockIdx.x, h = blockIdx.y * 16 + j;
  const bool h_ok = h < H;
  const int i = pos[t], slot = slot_[t];
  const int j_lo = i - window + 1 > 0 ? i - window + 1 : 0;
  const int total = i - j_lo + 1;
  const float scale2 = scale * LOG2E;
  const u16* kbase = reinterpret_cast<const u16*>(kv.k);
  u32x4 qf[NSM];
  f32x4 o[NVM];
  {
    const float* qr = qa + ((long)t * H + (h_ok ? h : H - 1)) * Dk;
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      const int d = 32 * s + 8 * g4;
      qf[s] = u32x4{0u, 0u, 0u, 0u};
      if (s < ns && d < Dk) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(qr + d), c = *reinterpret_cast<const f32x4*>(qr + d + 4);
        qf[s] = u32x4{pack2<P>(a[0], a[1]), pack2<P>(a[2], a[3]), pack2<P>(c[0], c[1]), pack2<P>(c[2], c[3])};
      }
    }
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  float m_run = -INFINITY, l_run = 0.f;
  const int nch = Dc >> 3;
  for (int base = wave * 32; base < total; base += 128) {
    if (lane < 32) {
      const int kx = base + lane;
      offs[lane] = kx < total ? pkv_tok(kv, slot, j_lo + kx, 0, 1, Dk) : -1;
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    {
      // lane = (key row m, parity of the 16-byte chunk); eight chunks of the row in flight before any is written
      const int m = lane & 31, c0 = lane >> 5;
      const long offm = offs[m];
      for (int cb = 0; cb < nch; cb += 16) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int ch = cb + c0 + 2 * u;
          v[u] = (ch < nch && offm >= 0) ? *reinterpret_cast<const u32x4*>(kbase + offm + 8 * ch) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int ch = cb + c0 + 2 * u;
          if (ch < nch) *reinterpret_cast<u32x4*>(v_s + m * LD + 8 * ch) = v[u];
        }
      }
    }
    f32x4 sc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      const long off = offs[16 * u + j];
      const u16* kr = kbase + (off >= 0 ? off : 0);
      u32x4 kf[NSM];
#pragma unroll
      for (int s = 0; s < NSM; ++s) {
        const int d = 32 * s + 8 * g4;
        kf[s] = (s < ns && d < Dk && off >= 0) ? *reinterpret_cast<const u32x4*>(kr + d) : u32x4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int s = 0; s < NSM; ++s) {
        if (s < ns) sc[u] = P::mfma(kf[s], qf[s], sc[u]);
      }
    }
    float sv[8], mx = -INFINITY;                                // maxima and exponents in base 2: one v_exp_f32 per weight
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const bool vis = base + 16 * u + 4 * g4 + rr < total;
        sv[4 * u + rr] = vis ? sc[u][rr] * scale2 : -INFINITY;
        mx = fmaxf(mx, sv[4 * u + rr]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);                       // finite: every step a wave runs has a key
    const float fac = __builtin_amdgcn_exp2f(m_run - m_new);
    float w[8], sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      w[e] = __builtin_amdgcn_exp2f(sv[e] - m_new);
      sum += w[e];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    l_run = l_run * fac + sum;
    m_run = m_new;
    if (__ballot(fac != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < NVM; ++dt) {
        if (dt < nv) { o[dt][0] *= fac; o[dt][1] *= fac; o[dt][2] *= fac; o[dt][3] *= fac; }
      }
    }
    const u32x4 pf = u32x4{pack2<P>(w[0], w[1]), pack2<P>(w[2], w[3]), pack2<P>(w[4], w[5]), pack2<P>(w[6], w[7])};
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) {
      if (dt < nv) {
        unsigned e[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) e[m] = v_s[((m >> 2) * 16 + 4 * g4 + (m & 3)) * LD + 16 * dt + j];
        const u32x4 va = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
        o[dt] = P::mfma(va, pf, o[dt]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  // merge the four waves: the value tiles are done with, their LDS holds [4][nv][64] partial tiles and [4][16] (max, sum)
  __syncthreads();
  f32x4* part = reinterpret_cast<f32x4*>(lat_lds);
  float* ml = reinterpret_cast<float*>(part + 4 * nv * 64);
#pragma unroll
  for (int dt = 0; dt < NVM; ++dt) {
    if (dt < nv) part[(wave * nv + dt) * 64 + lane] = o[dt];
  }
  if (g4 == 0) { ml[(wave * 16 + j) * 2] = m_run; ml[(wave * 16 + j) * 2 + 1] = l_run; }
  __syncthreads();
  if (!h_ok) return;
  const float sk = sink ? P::to_f(sink[h]) * LOG2E : -INFINITY;          // the running maxima are in base 2
  float M = sk, f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, ml[(w * 16 + j) * 2]);
  float L = sink ? exp2f(sk - M) : 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float mw = ml[(w * 16 + j) * 2];
    f[w] = mw == -INFINITY ? 0.f : exp2f(mw - M);
    L += ml[(w * 16 + j) * 2 + 1] * f[w];
  }
  const float inv = 1.f / L;
  for (int dt = wave; dt < nv; dt += 4) {
    f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const f32x4 pv = part[(w * nv + dt) * 64 + lane];
      a[0] += pv[0] * f[w]; a[1] += pv[1] * f[w]; a[2] += pv[2] * f[w]; a[3] += pv[3] * f[w];
    }
    u32x2 pk;
    pk[0] = pack2<P>(a[0] * inv, a[1] * inv);
    pk[1] = pack2<P>(a[2] * inv, a[3] * inv);
    *reinterpret_cast<u32x2*>(out + ((long)t * H + h) * Dc + 16 * dt + 4 * g4) = pk;
  }
}

extern "C" int umb_lat_attend_tiled_ok(int H, int kv_rank, int rot_dim, int dtype) {
  const int Dk = kv_rank + rot_dim;
  return H >= 1 && (dtype == UMB_SEQ_BF16 || dtype == UMB_SEQ_F16) && kv_rank >= 16 && kv_rank % 16 == 0 && kv_rank <= 512 &&
         rot_dim >= 0 && Dk % 8 == 0 && Dk <= 576;
}

extern "C" int umb_lat_attend_tiled(void* out, const float* qa, const UmbPagedKV* kv, const void* sink, const int* seq_slot,
                                    const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int max_len, int H,
                                    int kv_rank, int rot_dim, int window, float scale, int dtype, hipStream_t st) {
  if (B < 1 || max_len < 1 || window < 1 || !out || !qa || !lat_kv_ok(kv) || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len ||
      !umb_lat_attend_tiled_ok(H, kv_rank, rot_dim, dtype))
    return UMB_EINVAL;
  const int Dk = kv_rank + rot_dim;
  const size_t lds = ((size_t)32 * (Dk + 8) + (size_t)kv_rank * 36) * sizeof(u16);
#define LAT_MFMA(NSM, NVM, HPW)                                                                                            \
  do {                                                                                                                     \
    const dim3 grid((max_len + 15) / 16, B, (H + 4 * HPW - 1) / (4 * HPW));                                                \
    if (ensure_dynamic_lds<lat_attend_mfma_kernel<P, NSM, NVM, HPW>>(lds) != UMB_OK) return UMB_EHIP;                      \
    hipLaunchKernelGGL((lat_attend_mfma_kernel<P, NSM, NVM, HPW>), grid, dim3(256), lds, st, (u16*)out, qa, *kv,           \
                       (const u16*)sink, seq_slot, seq_row0, seq_pos0, seq_len, H, kv_rank, rot_dim, window, scale);       \
  } while (0)
#define LAT_MFMA_SHAPE()                                                                                                   \
  if (Dk <= 128 && kv_rank <= 128) { if (H >= 8) LAT_MFMA(4, 8, 2); else LAT_MFMA(4, 8, 1); }                              \
  else if (Dk <= 320 && kv_rank <= 256) LAT_MFMA(10, 16, 1);   /* two heads a wave spill to AGPRs here: measured slower */ \
  else LAT_MFMA(18, 32, 1)
  if (dtype == UMB_SEQ_BF16) { using P = BF16; LAT_MFMA_SHAPE(); }
  else { using P = F16; LAT_MFMA_SHAPE(); }
#undef LAT_MFMA_SHAPE
#undef LAT_MFMA
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_lat_prep(void* cq, const UmbPagedKV* kv, const float* proj, int ld, const void* w_q, const void* w_kv,
                            const int* pos, const int* slot, const float* freq, int T, int q_rank, int kv_rank, int rot_dim,
                            int rot_dims, float eps, int dtype, hipStream_t st) {
  if (T < 1 || q_rank < 1 || kv_rank < 1 || rot_dim < 0 || rot_dims < 0 || rot_dims > rot_dim || (rot_dims & 1) || !cq ||
      !lat_kv_ok(kv) || !proj || !w_q || !w_kv || !pos || !slot || (rot_dims && !freq) || ld < q_rank + kv_rank + rot_dim)
    return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(lat_prep_kernel<P>, dim3((unsigned)(2L * T)), dim3(256), 0, st, (E*)cq, *kv, proj, ld,
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
  // Few tokens: the vector-pipe kernel below spreads a token's keys over sixteen waves and its heads over several workgroups
  // and finishes sooner; from a few dozen tokens on the chip is full either way and sharing each key fragment among sixteen
  // heads wins (batch 128 at 1024 keys, kv_rank 512: 1.17 ms a step against 2.40).  UMB_LAT_DEC_MIN moves the switch.
  const char* env = getenv("UMB_LAT_DEC_MIN");
  const int lat_dec_min = env ? atoi(env) : 48;
  if (H >= 4 && T >= lat_dec_min && umb_lat_attend_tiled_ok(H, kv_rank, rot_dim, dtype)) {
    // 16-bit storage: sixteen heads of a token form the query tile of the matrix-pipe kernel
    const int Dk = kv_rank + rot_dim;
    const size_t tiles = 4 * (size_t)(32 * (kv_rank + 8) + 128) * sizeof(u16);
    const size_t parts = (size_t)4 * (kv_rank / 16) * 64 * sizeof(f32x4) + 4 * 16 * 2 * sizeof(float);
    const size_t lds = tiles > parts ? tiles : parts;
    const dim3 grid(T, (H + 15) / 16);
#define LAT_DEC(NSM, NVM)                                                                                                  \
  do {                                                                                                                     \
    if (ensure_dynamic_lds<lat_decode_mfma_kernel<P, NSM, NVM>>(lds) != UMB_OK) return UMB_EHIP;                           \
    hipLaunchKernelGGL((lat_decode_mfma_kernel<P, NSM, NVM>), grid, dim3(256), lds, st, (u16*)out, qa, *kv,                \
                       (const u16*)sink, pos, slot, H, kv_rank, rot_dim, window, scale);                                   \
  } while (0)
#define LAT_DEC_SHAPE()                                                                                                    \
  if (Dk <= 128 && kv_rank <= 128) LAT_DEC(4, 8); else if (Dk <= 320 && kv_rank <= 256) LAT_DEC(10, 16); else LAT_DEC(18, 32)
    if (dtype == UMB_SEQ_BF16) { using P = BF16; LAT_DEC_SHAPE(); }
    else { using P = F16; LAT_DEC_SHAPE(); }
#undef LAT_DEC_SHAPE
#undef LAT_DEC
    UMB_LAUNCH_CHECK();
    return UMB_OK;
  }
  const int Dk = kv_rank + rot_dim, Dp = (Dk + 3) & ~3;
  // heads of one workgroup: all of them share the keys, so as many as the register budget of the partial sums allows
  const int nc = (kv_rank + 63) / 64;
  int rh = nc <= 2 ? 8 : (nc <= 4 ? 4 : (nc <= 8 ? 2 : 1));
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
    else if (nc <= 8) { if (rh == 2) { LAT_NW(2, 8); } else { LAT_NW(1, 8); } }
    else { LAT_NW(1, 16); }
  })
#undef LAT_NW
#undef LAT_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

