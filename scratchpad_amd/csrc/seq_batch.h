// The requests of one step as the per-sequence state kernels see them: which request a token row belongs to, where the
// request's rows start, how many tokens it already holds.  A decode step (extend arrays null) has one row per request.
#pragma once
#include "sp_common.h"

namespace sp {

constexpr int kBlock = 256;

static __device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();                 // red may still be read from a previous call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) t += red[w];
  return t;
}

// ---- which token precedes each token of the step (for the bigram row and the token shift) ------------------------
// decode (extend arrays null): request b has one token at row b, prefix = seq_len - 1
struct SeqBatch {
  const void* req_pool_indices;
  const void* seq_lens;
  const int32_t* extend_seq_lens;
  const int32_t* extend_prefix_lens;
  const int32_t* extend_start_loc;
  const int32_t* token_req;
  int idx64;
  int B;
};
static __device__ __forceinline__ void seq_of_token(const SeqBatch& s, int64_t t, int& b, int64_t& start, int64_t& prefix) {
  if (s.extend_seq_lens) {
    b = s.token_req[t];
    start = s.extend_start_loc[b];
    prefix = s.extend_prefix_lens[b];
  } else {
    b = (int)t;
    start = t;
    prefix = load_idx(s.seq_lens, b, s.idx64) - 1;
  }
}
static __device__ __forceinline__ void seq_span(const SeqBatch& s, int b, int64_t& start, int64_t& len, int64_t& prefix) {
  if (s.extend_seq_lens) {
    start = s.extend_start_loc[b];
    len = s.extend_seq_lens[b];
    prefix = s.extend_prefix_lens[b];
  } else {
    start = b;
    len = 1;
    prefix = load_idx(s.seq_lens, b, s.idx64) - 1;
  }
}

}  // namespace sp

/* the struct made of an entry point's SP_SEQ_PARAMS */
#define SEQ_BATCH(name)                                                                                              \
  sp::SeqBatch name{req_pool_indices, seq_lens, extend_seq_lens, extend_prefix_lens, extend_start_loc, token_req, idx64, \
                batch_size}

