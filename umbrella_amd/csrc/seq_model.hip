// Forward pass of a sequence-mixer stack: walks the layer list of a UmbSeqModel and launches the kernels of
// seq_linear / seq_norm / seq_gla / seq_pwattn on one stream.  A layer is
//     x <- x + norm1b(mixer(norm1(x)))      x <- x + norm2b(ff(norm2(x)))    (the second only where the layer has one)
// with every norm a grouped RMS norm.  The seam kernel (resid_norm) adds a sublayer's normed output into the fp32 residual
// stream and produces the next sublayer's normed input in one pass, so a layer is
//     attention: proj GEMM | rope + unit-norm + append | pool | attend (matrix pipe for prompts) | out GEMM | seam | gate-up GEMM (SiLU*up epilogue) |
//                down GEMM | seam
//     GLA:       proj GEMM | decay | scan | head norm * SiLU gate | out GEMM | seam (| feed-forward as above)
// Nothing here depends on the host between launches: a step can be captured into a hipGraph.
#include "seq_common.h"

#define SEQ_TRY(call)            \
  do {                           \
    const int rc__ = (call);     \
    if (rc__ != UMB_OK) return rc__; \
  } while (0)

static inline int lin(const UmbSeqLinear& l, void* out, const void* x, int T, int epi, int dtype, hipStream_t st) {
  return umb_seq_linear(out, x, l.w, l.bias, T, l.N, l.K, epi, dtype, st);
}

static const void* first_norm_of(const UmbSeqModel* m, int l) { return l < m->L ? m->layers[l].norm1 : nullptr; }

extern "C" int umb_seq_forward(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  if (!m || !ws || !s || m->L < 1 || !m->layers || s->T < 1 || s->T > ws->Tmax || s->B < 1 || s->R < 0 || s->R > ws->Rmax)
    return UMB_EINVAL;
  const int T = s->T, W = m->W, dt = m->dtype, groups = m->groups;
  const float eps = m->eps;
  SEQ_TRY(umb_seq_embed_norm(ws->x, ws->h, m->embed, s->tokens, m->layers[0].norm1, T, W, m->V, groups, eps, dt, st));
  for (int l = 0; l < m->L; ++l) {
    const UmbSeqLayer& ly = m->layers[l];
    const int ld = ly.proj.N;
    SEQ_TRY(lin(ly.proj, ws->proj, ws->h, T, 0, dt, st));
    if (ly.kind == UMB_MIX_POOLED_WINDOW) {
      const int H = ly.heads, G = ly.kv_heads, D = ly.dim;
      if (ly.vdim != D || ld != H * D + G * D + H) return UMB_EINVAL;
      SEQ_TRY(umb_pwa_prep(ws->aux, &ly.kv, ws->proj, ld, s->pos, s->slot, ly.rot_freq, T, H, G, D, ly.rot_dims, eps, dt, st));
      SEQ_TRY(umb_pwa_pool(&ly.kv, s->seq_slot, s->seq_pos0, s->seq_len, s->B, s->max_len, G, D, ly.pool, dt, st));
      // steps that bring stretches of a sequence (prompts) take the matrix-pipe kernel where the shape allows it
      if (dt != UMB_SEQ_F32 && D % 32 == 0 && D <= 256 && s->max_len >= 16)
        SEQ_TRY(umb_pwa_attend_tiled(ws->mix, ws->aux, &ly.kv, ws->proj, ld, H * D + G * D, ly.pos_bias, s->seq_slot, s->seq_row0,
                                     s->seq_pos0, s->seq_len, s->B, s->max_len, H, G, D, ly.window, ly.pool, ly.scale, dt, st));
      else
        SEQ_TRY(umb_pwa_attend(ws->mix, ws->aux, &ly.kv, ws->proj, ld, H * D + G * D, ly.pos_bias, s->pos, s->slot, T, H, G, D,
                               ly.window, ly.pool, ly.scale, dt, st));
    } else if (ly.kind == UMB_MIX_GLA) {
      const int H = ly.heads, D = ly.dim, Dv = ly.vdim, HD = H * D;
      if (ld != 2 * HD + 2 * H * Dv + ly.rank || !ly.state) return UMB_EINVAL;
      SEQ_TRY(umb_gla_decay(ws->aux, ws->proj, ld, 2 * HD + 2 * H * Dv, ly.a2.w, ly.a2.bias, T, HD, ly.rank, ly.tau, dt, st));
      SEQ_TRY(umb_gla_scan(ws->o, ly.state, ws->proj, ld, ws->aux, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B, H, D,
                           Dv, ly.qscale, st));
      SEQ_TRY(umb_gla_gate(ws->mix, ws->o, ws->proj, ld, 2 * HD + H * Dv, ly.head_norm, T, H, Dv, eps, dt, st));
    } else {
      return UMB_EINVAL;
    }
    SEQ_TRY(lin(ly.out, ws->y, ws->mix, T, 0, dt, st));
    const void* next = ly.has_mlp ? ly.norm2 : first_norm_of(m, l + 1);
    SEQ_TRY(umb_seq_resid_norm(ws->x, ws->h, ws->y, ly.norm1b, next, T, W, groups, eps, dt, st));
    if (ly.has_mlp) {
      SEQ_TRY(lin(ly.gu, ws->act, ws->h, T, 2, dt, st));
      SEQ_TRY(lin(ly.down, ws->y, ws->act, T, 0, dt, st));
      SEQ_TRY(umb_seq_resid_norm(ws->x, ws->h, ws->y, ly.norm2b, first_norm_of(m, l + 1), T, W, groups, eps, dt, st));
    }
    if (s->trace) {
      if (hipMemcpyAsync(s->trace + (long)l * T * W, ws->x, (size_t)T * W * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
        return UMB_EHIP;
    }
  }
  if (s->R > 0) {
    // final norm of the wanted rows only, then the head
    SEQ_TRY(umb_seq_group_norm(nullptr, ws->h, ws->x, s->logit_rows, m->final_norm, s->R, W, groups, eps, dt, st));
    SEQ_TRY(lin(m->head, ws->logits, ws->h, s->R, 0, dt, st));
  }
  return UMB_OK;
}

extern "C" const char* umb_seq_version(void) { return "umbrella_seq 0.1 (gfx950)"; }
