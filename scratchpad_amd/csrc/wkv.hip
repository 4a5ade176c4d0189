// Linear-recurrence mixer with a per-head matrix state (RWKV-style time mixing):
//   token shift      m_s[t] = h[t] + (h[t-1] - h[t]) * mu_s            (h[-1] = the sequence's saved row, or zeros)
//   decay            w[t]   = exp(-exp(W2 tanh(a[t]) + w0))            (a = the low-rank projection's output)
//   recurrence       o[t]   = (S + diag(u) k v^T)^T r ;  S <- diag(w) S + k v^T      (S: key channel x value channel)
//   output           o / rms_head(o) * norm * silu(g)
// State, decays and the recurrence are fp32 whatever the projections' element type.
//
// The recurrence runs one workgroup per (request, head): thread j owns value column j of S in registers, the step's
// r / k / w / u are broadcast from LDS, and the request's tokens of this step are walked in order from the state the
// previous step left in the pool (zeros at a sequence's first token).  Requests with one token (decode) and with many
// (a prompt's portion) take the same path.
#include "seq_batch.h"

namespace sp {
namespace {

template <typename Tag>
__global__ void token_shift_kernel(void* out, const float* x, const float* mu, const float* shift_state,
                                   int64_t state_stride, SeqBatch s, int64_t T, int width, int mixes, int64_t x_stride) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const float* prev = nullptr;
  if (t > start) prev = x + (t - 1) * x_stride;
  else if (prefix > 0) prev = shift_state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float h = x[t * x_stride + i];
    const float d = (prev ? prev[i] : 0.f) - h;
    for (int m = 0; m < mixes; ++m) E::store(out, ((int64_t)m * T + t) * width + i, h + d * mu[(int64_t)m * width + i]);
  }
}

// w2t: [rank, channels] fp32 (the up-projection transposed: neighbouring threads read neighbouring channels)
template <typename Tag>
__global__ void wkv_decay_kernel(float* decay, const void* a, const float* w2t, const float* w0, int channels, int rank,
                                 int64_t a_stride) {
  typedef Elem<Tag> E;
  extern __shared__ float ta[];
  const int64_t t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += blockDim.x) ta[r] = tanhf(E::load(a, t * a_stride + r));
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float acc = w0[c];
    for (int r = 0; r < rank; ++r) acc += w2t[(int64_t)r * channels + c] * ta[r];
    decay[t * channels + c] = expf(-expf(acc));
  }
}

constexpr int kChunk = 8;       // tokens staged in LDS per pass

template <typename Tag, int KP>      // KP: head size rounded up to a power of two (register file of the state column)
__global__ void __launch_bounds__(KP < 64 ? 64 : KP)
wkv_recurrence_kernel(void* out, const void* r, const void* k, const void* v, const void* g, const float* decay,
                      const float* u, const float* norm_w, float* state, int64_t state_stride, SeqBatch s, int H, int K,
                      int64_t rs, int64_t ks, int64_t vs, int64_t gs, int64_t os, float eps) {
  typedef Elem<Tag> E;
  __shared__ float sr[kChunk][KP], sk[kChunk][KP], sw[kChunk][KP], so[kChunk][KP], su[KP];
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int nthreads = blockDim.x;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = j < K;
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride + (int64_t)h * K * K;
  float S[KP];
#pragma unroll
  for (int i = 0; i < KP; ++i) S[i] = (live && i < K && prefix > 0) ? st[(int64_t)i * K + j] : 0.f;
  for (int i = j; i < KP; i += nthreads) su[i] = i < K ? u[h * K + i] : 0.f;
  const int64_t col = (int64_t)h * K;
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();
    for (int e = j; e < n * KP; e += nthreads) {
      const int tt = e / KP, i = e % KP;
      const int64_t row = start + c0 + tt;
      const bool ok = i < K;
      sr[tt][i] = ok ? E::load(r, row * rs + col + i) : 0.f;
      sk[tt][i] = ok ? E::load(k, row * ks + col + i) : 0.f;
      sw[tt][i] = ok ? decay[row * ((int64_t)H * K) + col + i] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float vj = live ? E::load(v, (start + c0 + tt) * vs + col + j) : 0.f;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KP; ++i) {
        const float kv = sk[tt][i] * vj;
        o += sr[tt][i] * (S[i] + su[i] * kv);
        S[i] = sw[tt][i] * S[i] + kv;
      }
      if (j < KP) so[tt][j] = live ? o : 0.f;
    }
    __syncthreads();
    // per-head RMS of o, output weight and gate: one wave per token of the pass
    const int wave = j >> 6, lane = j & 63, waves = nthreads >> 6;
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < K; i += 64) ss += so[tt][i] * so[tt][i];
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)K + eps);
      const int64_t row = start + c0 + tt;
      for (int i = lane; i < K; i += 64) {
        const float gv = E::load(g, row * gs + col + i);
        const float gate = gv / (1.f + expf(-gv));
        E::store(out, row * os + col + i, so[tt][i] * inv * norm_w[col + i] * gate);
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (i < K) st[(int64_t)i * K + j] = S[i];
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_token_shift(void* out, const float* x, const float* mu, const float* shift_state, int64_t state_stride,
                              int64_t num_tokens, int width, int mixes, int64_t x_stride, SP_SEQ_PARAMS, int dtype,
                              void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && mixes > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && x && mu && shift_state && req_pool_indices && seq_lens && x_stride >= width && state_stride >= width);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, (token_shift_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               out, x, mu, shift_state, state_stride, s, num_tokens, width, mixes, x_stride)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_wkv_decay(float* decay, const void* a, const float* w2t, const float* w0, int64_t num_tokens,
                            int channels, int rank, int64_t a_stride, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && channels > 0 && rank > 0 && rank <= 8192);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(decay && a && w2t && w0 && a_stride >= rank);
  SP_DISPATCH_DTYPE(dtype, (wkv_decay_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, rank * sizeof(float),
                                                     (hipStream_t)stream>>>(decay, a, w2t, w0, channels, rank, a_stride)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

template <typename Tag>
static int launch_wkv(void* out, const void* r, const void* k, const void* v, const void* g, const float* decay,
                      const float* u, const float* norm_w, float* state, int64_t state_stride, const SeqBatch& s, int H,
                      int K, int64_t rs, int64_t ks, int64_t vs, int64_t gs, int64_t os, float eps, hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
#define SP_WKV(KP)                                                                                                    \
  wkv_recurrence_kernel<Tag, KP><<<grid, (KP < 64 ? 64 : KP), 0, st>>>(out, r, k, v, g, decay, u, norm_w, state,      \
                                                                       state_stride, s, H, K, rs, ks, vs, gs, os, eps)
  if (K <= 16) SP_WKV(16);
  else if (K <= 32) SP_WKV(32);
  else if (K <= 64) SP_WKV(64);
  else if (K <= 128) SP_WKV(128);
  else if (K <= 256) SP_WKV(256);
  else return SP_ERR_UNSUPPORTED;
#undef SP_WKV
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_wkv_recurrence(void* out, const void* r, const void* k, const void* v, const void* g,
                                 const float* decay, const float* u, const float* norm_w, float* state,
                                 int64_t state_stride, int heads, int head_dim, int64_t r_stride, int64_t k_stride,
                                 int64_t v_stride, int64_t g_stride, int64_t out_stride, float eps, SP_SEQ_PARAMS,
                                 int dtype, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && head_dim > 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(out && r && k && v && g && decay && u && norm_w && state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SP_CHECK_ARG(state_stride >= (int64_t)heads * head_dim * head_dim);
  const int64_t n = (int64_t)heads * head_dim;
  SP_CHECK_ARG(r_stride >= n && k_stride >= n && v_stride >= n && g_stride >= n && out_stride >= n);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_wkv<Tag>(out, r, k, v, g, decay, u, norm_w, state, state_stride, s, heads,
                                                   head_dim, r_stride, k_stride, v_stride, g_stride, out_stride, eps,
                                                   (hipStream_t)stream)));
}
