// Shared helpers of the sequence-mixer kernels (libumbrella_seq.so): a third storage policy (fp32) beside the 16-bit ones
// of common.h, typed element access, and the paged key/value addressing.
#pragma once
#include "common.h"
#include "../../include/umbrella_seq.h"

struct F32 {};

template <typename P> struct El { typedef u16 type; };
template <> struct El<F32> { typedef float type; };

template <typename P> __device__ __forceinline__ float ldf(const typename El<P>::type* p) { return P::to_f(*p); }
template <> __device__ __forceinline__ float ldf<F32>(const float* p) { return *p; }
template <typename P> __device__ __forceinline__ void stf(typename El<P>::type* p, float v) { *p = P::from_f(v); }
template <> __device__ __forceinline__ void stf<F32>(float* p, float v) { *p = v; }

#define DISPATCH_SEQ_DTYPE(dt, ...)                          \
  if ((dt) == UMB_SEQ_BF16) { using P = BF16; __VA_ARGS__ }  \
  else if ((dt) == UMB_SEQ_F16) { using P = F16; __VA_ARGS__ } \
  else if ((dt) == UMB_SEQ_F32) { using P = F32; __VA_ARGS__ } \
  else return UMB_EINVAL;

static inline size_t seq_elem_bytes(int dt) { return dt == UMB_SEQ_F32 ? 4 : 2; }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }
// log(sigmoid(x)) without overflow on either side
__device__ __forceinline__ float log_sigmoidf_(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }

// ---- paged key/value store: element offsets (in elements) of one token's / one pooled block's D-vector
__device__ __forceinline__ long pkv_tok(const UmbPagedKV& kv, int slot, int pos, int g, int G, int D) {
  const int pg = kv.pages[(long)slot * kv.max_pages + pos / kv.page];
  return (((long)pg * G + g) * kv.page + pos % kv.page) * D;
}
__device__ __forceinline__ long pkv_blk(const UmbPagedKV& kv, int slot, int b, int pool, int g, int G, int D) {
  const int e = b * pool + pool - 1;                      // the block's last position
  const int pg = kv.pages[(long)slot * kv.max_pages + e / kv.page];
  const int npb = (kv.page + pool - 1) / pool;
  return (((long)pg * G + g) * npb + (e % kv.page) / pool) * D;
}

// Dynamic LDS above the default limit needs the function attribute.  It is set once per kernel and size (a function-local
// static per kernel instantiation), i.e. by the first eager launch: a step that is being captured into a hipGraph has run
// eagerly before and makes no such call.
template <auto Kernel> static inline int ensure_dynamic_lds(size_t bytes) {
  static size_t granted = 48 * 1024;
  if (bytes > granted) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
      return UMB_EHIP;
    granted = bytes;
  }
  return UMB_OK;
}
