/* libumbrella_seq.so -- C ABI of the sequence-mixer model family on MI355X (gfx950).
 *
 * Decoder stacks whose layers mix tokens with something other than the dense tree-masked softmax attention of
 * libumbrella_hip.so: gated linear attention (a per-head matrix state carried from token to token) and sliding-window
 * attention over a paged key/value store with mean-pooled blocks behind the window and sigmoid (un-normalised) weights.
 * The layer list, every size and every constant are data (UmbSeqLayer); one forward entry point walks the list.
 *
 * Conventions are those of umbrella_hip.h: extern "C", plain pointers and sizes, 0 or a negative errno-style code,
 * nothing allocated, every call asynchronous on `stream`, all run-time indices read from device memory.
 *
 * dtype: 0 = fp16, 1 = bf16, 2 = fp32 -- the type of weights, of activations that feed a matrix product and of cached
 * keys / values.  Whatever the dtype, these are fp32: the residual stream, every norm, rotary angles, attention scores
 * and weights, decays, the recurrent state and everything that enters the recurrence, all matrix-product accumulators.
 *
 * A step is a RAGGED batch: T rows, the rows of one sequence contiguous and at consecutive positions.  Nothing is padded.
 */
#ifndef UMBRELLA_SEQ_H
#define UMBRELLA_SEQ_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* umb_stream_t;   /* == hipStream_t */

enum { UMB_SEQ_F16 = 0, UMB_SEQ_BF16 = 1, UMB_SEQ_F32 = 2 };
enum { UMB_MIX_POOLED_WINDOW = 0, UMB_MIX_GLA = 1 };

/* W [N][K] row-major (as stored: out x in), optional bias [N]; applied as W x + b */
typedef struct UmbSeqLinear { const void* w; const void* bias; int32_t N, K; } UmbSeqLinear;

/* ------------------------------------------------------------------ stand-alone ops (each is also a step of the forward) */

/* out[T][N] = x[T][K] . W^T + bias, fp32 accumulation in a fixed order that depends on (N, K) only.
 * epi 0: out fp32; epi 1: out in `dtype`; epi 2: W stacks [gate; up] (N = 2 N'), out[T][N'] in `dtype` =
 * silu(gate) * up.  x and W in `dtype`. */
int umb_seq_linear(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, int dtype,
                   umb_stream_t stream);

/* RMS norm in `groups` equal consecutive parts of a row: part / sqrt(mean(part^2) + eps), whole row times w.
 * x fp32 [*][W]; rows: optional gather (row i of out comes from row rows[i] of x); out_f32 and/or out_dt may be given. */
int umb_seq_group_norm(float* out_f32, void* out_dt, const float* x, const int* rows, const void* w, int T, int W, int groups,
                       float eps, int dtype, umb_stream_t stream);
/* x[t] <- embed[tokens[t]] (fp32); h[t] <- group_norm(x[t]) * w in `dtype` */
int umb_seq_embed_norm(float* x, void* h, const void* embed, const int* tokens, const void* w, int T, int W, int V, int groups,
                       float eps, int dtype, umb_stream_t stream);
/* x <- x + group_norm(y) * w_post ; if w_next: h <- group_norm(x) * w_next in `dtype`   (y fp32 [T][W]) */
int umb_seq_resid_norm(float* x, void* h, const float* y, const void* w_post, const void* w_next, int T, int W, int groups,
                       float eps, int dtype, umb_stream_t stream);

/* ---- gated linear attention.  proj fp32 [T][ld]: columns [q (H D) | k (H D) | v (H Dv) | g (H Dv) | a (rank)].
 * decay: alpha[t][H D] = sigmoid(W_a2 a + b)^(1/tau), fp32 */
int umb_gla_decay(float* alpha, const float* proj, int ld, int a_col, const void* w_a2, const void* b_a2, int T, int HD, int rank,
                  float tau, int dtype, umb_stream_t stream);
/* per sequence and head: S <- diag(alpha_t) S + k_t v_t^T ; o_t = S^T (q_t * qscale).  state fp32 [slots][H][D][Dv]; a
 * sequence whose first position is 0 starts from S = 0 whatever its slot holds.  o fp32 [T][H Dv]. */
int umb_gla_scan(float* o, float* state, const float* proj, int ld, const float* alpha, const int* seq_slot, const int* seq_row0,
                 const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv, float qscale, umb_stream_t stream);
/* out[t][h] = rms_norm(o[t][h]) * w (w [Dv], shared by heads) * silu(g[t][h]) in `dtype` */
int umb_gla_gate(void* out, const float* o, const float* proj, int ld, int g_col, const void* w, int T, int H, int Dv, float eps,
                 int dtype, umb_stream_t stream);

/* ---- sliding-window attention with pooled blocks over a paged store.
 * Pages hold `page` tokens; page table pages[slot][max_pages].  Per layer: K and V [pages][G][page][D] in `dtype`, and
 * the pooled K / V [pages][G][ceil(page / pool)][D] in fp32: block b (positions b pool .. b pool + pool - 1) lives in the
 * page of its LAST position e, at entry (e % page) / pool. */
typedef struct UmbPagedKV {
  void* k; void* v; float* kp; float* vp;
  const int32_t* pages; int32_t max_pages, page, n_pages, pad_;
} UmbPagedKV;
/* proj fp32 [T][ld]: columns [q (H D) | k (G D) | gate (H)] with the projection biases already added.
 * q <- unit_rms(rope(q)) fp32 [T][H D]; cache K <- unit_rms(rope(k)), cache V <- k as projected; interleaved pairs
 * (2i, 2i+1) of the first rot_dims features turn by pos * freq[i]. */
int umb_pwa_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const int* pos, const int* slot, const float* freq,
                 int T, int H, int G, int D, int rot_dims, float eps, int dtype, umb_stream_t stream);
/* pooled entries of every block whose last position this step wrote: the fp32 mean of the `pool` cached keys / values */
int umb_pwa_pool(const UmbPagedKV* kv, const int* seq_slot, const int* seq_pos0, const int* seq_len, int B, int max_len, int G,
                 int D, int pool, int dtype, umb_stream_t stream);
/* out[t][h] = sigmoid(gate[t][h]) * sum over visible keys of sigmoid(q.k * scale + pos_bias[h]) * v, in `dtype`.
 * Visible to position i: tokens j with 0 <= i - j < window, and blocks b with b pool + pool - 1 <= i - window. */
int umb_pwa_attend(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col, const void* pos_bias,
                   const int* pos, const int* slot, int T, int H, int G, int D, int window, int pool, float scale, int dtype,
                   umb_stream_t stream);

/* The same attention for steps that bring whole stretches of a sequence (prompts), on the matrix pipe: 16-bit storage only,
 * D a multiple of 32 (<= 256); workgroups own 16 consecutive positions of one sequence.  Scores and weights keep fp32
 * accuracy: the fp32 factors (q, pooled means, weights) enter as high + low 16-bit halves. */
int umb_pwa_attend_tiled(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                         const void* pos_bias, const int* seq_slot, const int* seq_row0, const int* seq_pos0, const int* seq_len,
                         int B, int max_len, int H, int G, int D, int window, int pool, float scale, int dtype,
                         umb_stream_t stream);

/* ------------------------------------------------------------------ the model */
typedef struct UmbSeqLayer {
  int32_t kind, has_mlp;
  int32_t heads, kv_heads, dim, vdim;
  int32_t window, pool, rot_dims, rank;
  int32_t ff, pad_;
  float scale, tau, qscale, pad2_;
  UmbSeqLinear proj;      /* fused input projection: [q | k | gate] or [q | k | v | g | a] */
  UmbSeqLinear a2;        /* GLA: decay up-projection [heads dim][rank] + bias */
  UmbSeqLinear out;       /* output projection */
  UmbSeqLinear gu, down;  /* feed-forward: stacked [gate; up], down */
  const void* pos_bias;   /* attention: [heads] */
  const void* head_norm;  /* GLA: [vdim] */
  const void *norm1, *norm1b, *norm2, *norm2b;
  const float* rot_freq;  /* [rot_dims / 2] fp32 */
  UmbPagedKV kv;          /* attention layers */
  float* state;           /* GLA layers: [slots][heads][dim][vdim] fp32 */
} UmbSeqLayer;

typedef struct UmbSeqModel {
  int32_t dtype, L, W, V, groups, pad_;
  float eps, pad2_;
  const void* embed; const void* final_norm; UmbSeqLinear head;
  const UmbSeqLayer* layers;
} UmbSeqModel;

/* activations of one step (caller-owned, sized for Tmax rows) */
typedef struct UmbSeqWork {
  float* x;        /* residual stream [Tmax][W] fp32 */
  void* h;         /* normed input of the current sublayer [Tmax][W] dtype */
  float* proj;     /* fused projection output [Tmax][max proj N] fp32 */
  float* aux;      /* q / alpha [Tmax][max heads*dim] fp32 */
  float* o;        /* GLA scan output [Tmax][max heads*vdim] fp32 */
  void* mix;       /* mixer output before the output projection [Tmax][max heads*vdim] dtype */
  void* act;       /* feed-forward activation [Tmax][max ff] dtype */
  float* y;        /* sublayer output [Tmax][W] fp32 */
  float* logits;   /* [Rmax][V] fp32 */
  int32_t Tmax, Rmax;
} UmbSeqWork;

typedef struct UmbSeqStep {
  int32_t T, B, R, max_len;
  const int32_t *tokens, *pos, *slot;                       /* [T] */
  const int32_t *seq_slot, *seq_row0, *seq_pos0, *seq_len;  /* [B] */
  const int32_t* logit_rows;                                /* [R] rows whose logits are wanted */
  float* trace;                                             /* optional [L][T][W]: the residual stream after every layer */
} UmbSeqStep;

int umb_seq_forward(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, umb_stream_t stream);

/* sampling on fp32 logits rows (the same kernels as libumbrella_hip.so) */
int umb_argmax_rows(int* out, const float* logits, int rows, int V, umb_stream_t stream);
int umb_sample_rows(int* sampled, float* logits, int rows, int V, const int* tokens_all, const int* n_ptr,
                    float penalty, float temperature, int topk, float topp, const void* seed, int dbg_k,
                    int* dbg_idx, float* dbg_p, umb_stream_t stream);

const char* umb_seq_version(void);

#ifdef __cplusplus
}
#endif
#endif
