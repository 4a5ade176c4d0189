// Residual stream kept in fp32 with single-gain RMS norms on the sublayer OUTPUT (x += norm(f(x)) * g), the hashed
// bigram embedding, PolyNorm, per-head output gates, and the row saves of per-sequence state.
//
// Every kernel here takes one workgroup per token (or per request) and reduces in fp32.  Activations that feed a
// projection are written in the projection's element type next to the fp32 stream, so no separate cast runs.
#include "seq_batch.h"

namespace sp {
namespace {

__global__ void bigram_rows_kernel(int32_t* rows, const int64_t* ids, const int64_t* last_token, SeqBatch s, int64_t T,
                                   int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  int64_t prev;
  if (t > start) prev = ids[t - 1];
  else prev = prefix > 0 ? last_token[load_idx(s.req_pool_indices, b, s.idx64)] : -1;
  rows[t] = prev < 0 ? (int32_t)buckets : (int32_t)((prev * mul_prev + ids[t] * mul_cur) % buckets);
}

__global__ void save_last_token_kernel(int64_t* last_token, const int64_t* ids, SeqBatch s) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= s.B) return;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len > 0) last_token[load_idx(s.req_pool_indices, b, s.idx64)] = ids[start + len - 1];
}

// state[slot(b), :] = x[last token of b, :]
__global__ void save_last_rows_kernel(float* state, int64_t state_stride, const float* x, int64_t x_stride, int width,
                                      SeqBatch s) {
  const int b = blockIdx.x;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const float* src = x + (start + len - 1) * x_stride;
  float* dst = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

// ---- x = norm(embed[id] + bigram[row]) * g ------------------------------------------------------------------------
template <typename Tag>
__global__ void embed_bigram_norm_kernel(float* x, void* lo, const void* embed, const void* bigram, const int64_t* ids,
                                         const int32_t* rows, const float* gain, int width, int64_t x_stride,
                                         int64_t lo_stride, float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  const int64_t e0 = ids[t] * (int64_t)width, b0 = (int64_t)rows[t] * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = E::load(embed, e0 + i) + E::load(bigram, b0 + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float scale = gain[0] / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = (E::load(embed, e0 + i) + E::load(bigram, b0 + i)) * scale;
    x[t * x_stride + i] = v;
    if (lo) E::store(lo, t * lo_stride + i, v);
  }
}

// ---- ADD: x += y / rms(y) * g (x fp32 in place), lo = x in the projections' type
//      else: lo = x / rms(x) * g (the model's final norm)
template <typename Tag, bool ADD>
__global__ void scalar_norm_kernel(float* x, void* lo, const void* y, const float* gain, int width, int64_t x_stride,
                                   int64_t lo_stride, int64_t y_stride, float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = ADD ? E::load(y, t * y_stride + i) : x[t * x_stride + i];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float scale = gain[0] / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    if (ADD) {
      const float v = x[t * x_stride + i] + E::load(y, t * y_stride + i) * scale;
      x[t * x_stride + i] = v;
      if (lo) E::store(lo, t * lo_stride + i, v);
    } else {
      E::store(lo, t * lo_stride + i, x[t * x_stride + i] * scale);
    }
  }
}

// ---- PolyNorm: a N(z) + b N(z^2) + c N(z^3) + e, N = division by the root mean square over the row ------------------
template <typename Tag>
__global__ void polynorm_kernel(void* out, const void* z, const float* coef, int n, int64_t z_stride, int64_t out_stride,
                                float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = E::load(z, t * z_stride + i);
    const float v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  s3 = block_sum(s3, red);
  const float a = coef[0] / sqrtf(s1 / (float)n + eps), b = coef[1] / sqrtf(s2 / (float)n + eps),
              c = coef[2] / sqrtf(s3 / (float)n + eps), e = coef[3];
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = E::load(z, t * z_stride + i);
    E::store(out, t * out_stride + i, a * v + b * v * v + c * v * v * v + e);
  }
}

// ---- out[t, h, :] = o[h, t, :] * sigmoid(g[t, h]) -----------------------------------------------------------------
template <typename Tag>
__global__ void gate_heads_kernel(void* out, const void* o, const void* g, int64_t T, int H, int D, int64_t g_stride) {
  typedef Elem<Tag> E;
  const int64_t n = T * H * (int64_t)D;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int d = (int)(i % D);
    const int h = (int)((i / D) % H);
    const int64_t t = i / ((int64_t)D * H);
    const float gate = 1.f / (1.f + expf(-E::load(g, t * g_stride + h)));
    E::store(out, i, E::load(o, ((int64_t)h * T + t) * D + d) * gate);
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_bigram_rows(int32_t* rows, const int64_t* ids, const int64_t* last_token, int64_t num_tokens,
                              SP_SEQ_PARAMS, int64_t buckets, int64_t mul_prev,
                              int64_t mul_cur, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && batch_size >= 0 && buckets > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(rows && ids && last_token && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SEQ_BATCH(s);
  bigram_rows_kernel<<<dim3((unsigned)((num_tokens + 255) / 256)), 256, 0, (hipStream_t)stream>>>(
      rows, ids, last_token, s, num_tokens, buckets, mul_prev, mul_cur);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_save_last_token(int64_t* last_token, const int64_t* ids, SP_SEQ_PARAMS, void* stream) {
  SP_CHECK_ARG(batch_size >= 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(last_token && ids && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SEQ_BATCH(s);
  save_last_token_kernel<<<dim3((unsigned)((batch_size + 255) / 256)), 256, 0, (hipStream_t)stream>>>(last_token, ids, s);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_save_last_rows(float* state, int64_t state_stride, const float* x, int64_t x_stride, int width,
                                 SP_SEQ_PARAMS, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && width > 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(state && x && req_pool_indices && seq_lens && state_stride >= width && x_stride >= width);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SEQ_BATCH(s);
  save_last_rows_kernel<<<dim3((unsigned)batch_size), kBlock, 0, (hipStream_t)stream>>>(state, state_stride, x, x_stride,
                                                                                       width, s);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_embed_bigram_norm(float* x, void* lo, const void* embed, const void* bigram, const int64_t* ids,
                                    const int32_t* rows, const float* gain, int64_t num_tokens, int width,
                                    int64_t x_stride, int64_t lo_stride, float eps, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && embed && bigram && ids && rows && gain && x_stride >= width && (!lo || lo_stride >= width));
  SP_DISPATCH_DTYPE(dtype, (embed_bigram_norm_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               x, lo, embed, bigram, ids, rows, gain, width, x_stride, lo_stride, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_add_scalar_norm(float* x, void* lo, const void* y, const float* gain, int64_t num_tokens, int width,
                                  int64_t x_stride, int64_t lo_stride, int64_t y_stride, float eps, int dtype,
                                  void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && y && gain && x_stride >= width && y_stride >= width && (!lo || lo_stride >= width));
  SP_DISPATCH_DTYPE(dtype, (scalar_norm_kernel<Tag, true><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               x, lo, y, gain, width, x_stride, lo_stride, y_stride, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_scalar_norm(void* out, const float* x, const float* gain, int64_t num_tokens, int width,
                              int64_t x_stride, int64_t out_stride, float eps, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && x && gain && x_stride >= width && out_stride >= width);
  SP_DISPATCH_DTYPE(dtype, (scalar_norm_kernel<Tag, false><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               (float*)x, out, nullptr, gain, width, x_stride, out_stride, 0, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_polynorm(void* out, const void* z, const float* coef, int64_t num_tokens, int n, int64_t z_stride,
                           int64_t out_stride, float eps, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && n > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && z && coef && z_stride >= n && out_stride >= n);
  SP_DISPATCH_DTYPE(dtype, (polynorm_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               out, z, coef, n, z_stride, out_stride, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_gate_heads(void* out, const void* o, const void* g, int64_t num_tokens, int heads, int head_dim,
                             int64_t g_stride, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && heads > 0 && head_dim > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && o && g && g_stride >= heads);
  int64_t blocks = (num_tokens * heads * head_dim + kBlock - 1) / kBlock;
  if (blocks > 4096) blocks = 4096;
  SP_DISPATCH_DTYPE(dtype, (gate_heads_kernel<Tag><<<dim3((unsigned)blocks), kBlock, 0, (hipStream_t)stream>>>(
                               out, o, g, num_tokens, heads, head_dim, g_stride)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}
