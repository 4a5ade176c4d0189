// Attention over a compressed (latent) key/value cache.  Per token the pool holds ONE row [c | k_rot]: the normed
// latent c (rank C) from which every head's unrotated key W_uk c and value W_uv c derive, and the rotated key part
// (R dimensions) all heads share.  The up-projections are folded into the query and the output:
//   score(t, s, h) = (W_uk_h^T q_h[t]) . c[s] + q_rot_h[t] . k_rot[s]          out_h[t] = W_uv_h (sum_s p(t, s, h) c[s])
// so the kernel is multi-query attention with key width C + R and value width C over the pool's rows; the caller
// runs the two per-head products as batched matrix products around it.
//
// Rotation: interleaved pairs (2i, 2i+1), angle = position * frequency[i] in fp32, cos and sin scaled by `mag`
// (frequency table and magnitude are the caller's: plain, or YaRN-blended).
#include "seq_batch.h"

namespace sp {
namespace {

// in place on x[t, h, offset + 0 .. R) for every head
template <typename Tag>
__global__ void rotary_interleaved_kernel(void* x, const int64_t* positions, const float* freq, float mag, int H, int R,
                                          int64_t token_stride, int64_t head_stride, int offset) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = R / 2;
  for (int e = threadIdx.x; e < H * half; e += blockDim.x) {
    const int h = e / half, i = e % half;
    const float a = pos * freq[i];
    const float c = cosf(a) * mag, s = sinf(a) * mag;
    const int64_t at = t * token_stride + (int64_t)h * head_stride + offset + 2 * i;
    const float u = E::load(x, at), v = E::load(x, at + 1);
    E::store(x, at, u * c - v * s);
    E::store(x, at + 1, v * c + u * s);
  }
}

// pool[loc[t]] = [ rmsnorm(dkv[t, :C]) * w | rotate(dkv[t, C:C+R]) ]   (the first rot_dims of the R rotate, the rest pass)
template <typename Tag>
__global__ void latent_kv_store_kernel(void* pool, int64_t pool_stride, const void* dkv, int64_t dkv_stride,
                                       const float* norm_w, const int64_t* positions, const float* freq, float mag,
                                       const int64_t* loc, int C, int R, int rot_dims, float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  const int64_t src = t * dkv_stride, dst = loc[t] * pool_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const float v = E::load(dkv, src + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)C + eps);
  for (int i = threadIdx.x; i < C; i += blockDim.x) E::store(pool, dst + i, E::load(dkv, src + i) * inv * norm_w[i]);
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
    const float a = pos * freq[i];
    const float c = cosf(a) * mag, s = sinf(a) * mag;
    const float u = E::load(dkv, src + C + 2 * i), v = E::load(dkv, src + C + 2 * i + 1);
    E::store(pool, dst + C + 2 * i, u * c - v * s);
    E::store(pool, dst + C + 2 * i + 1, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < R; i += blockDim.x) E::store(pool, dst + C + i, E::load(dkv, src + C + i));
}

constexpr int kMaxPerLane = 16;      // value width C <= 64 * kMaxPerLane

// One wave per (token, head); 4 heads of a token per workgroup.  Keys in tiles of 64: lane = key for the scores,
// lane = value channel for the weighted sum; running maximum and sum in fp32.
template <typename Tag>
__global__ void __launch_bounds__(256)
latent_attention_kernel(void* out, const void* q_lat, const void* q_rot, const void* pool, int64_t pool_stride,
                        const int32_t* req_to_token, int64_t table_stride, SeqBatch s, int64_t T, int H, int C, int R,
                        int64_t qrot_token_stride, int64_t qrot_head_stride, float scale) {
  typedef Elem<Tag> E;
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y * 4 + wave;
  if (h >= H) return;                                    // (no workgroup barrier below)
  float* sq = smem + (size_t)wave * (C + R + 64);        // this wave's query [C + R], then its 64 weights
  float* sp_ = sq + C + R;
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const int64_t keys = prefix + (t - start) + 1;        // positions 0 .. own
  const int32_t* table = req_to_token + load_idx(s.req_pool_indices, b, s.idx64) * table_stride;
  for (int i = lane; i < C; i += 64) sq[i] = E::load(q_lat, ((int64_t)h * T + t) * C + i) * scale;
  for (int i = lane; i < R; i += 64) sq[C + i] = E::load(q_rot, t * qrot_token_stride + (int64_t)h * qrot_head_stride + i) * scale;
  __builtin_amdgcn_wave_barrier();
  float m = -INFINITY, l = 0.f;
  float acc[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) acc[i] = 0.f;
  const int W = C + R;
  for (int64_t k0 = 0; k0 < keys; k0 += 64) {
    const int n = (int)(keys - k0 < 64 ? keys - k0 : 64);
    float sc = -INFINITY;
    int64_t row = 0;
    if (lane < n) {
      row = (int64_t)table[k0 + lane] * pool_stride;
      float d = 0.f;
      for (int i = 0; i < W; ++i) d += sq[i] * E::load(pool, row + i);
      sc = d;
    }
    float tm = sc;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) tm = fmaxf(tm, __shfl_xor(tm, off, 64));
    const float m_new = fmaxf(m, tm);
    const float corr = expf(m - m_new);                 // first tile: exp(-inf) = 0
    const float p = lane < n ? expf(sc - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    m = m_new;
    sp_[lane] = p;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) acc[i] *= corr;
    for (int j = 0; j < n; ++j) {
      const int64_t rj = (int64_t)table[k0 + j] * pool_stride;
      const float pj = sp_[j];
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int c = lane + 64 * i;
        if (c < C) acc[i] += pj * E::load(pool, rj + c);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int c = lane + 64 * i;
    if (c < C) E::store(out, ((int64_t)h * T + t) * C + c, acc[i] * inv);
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_rotary_interleaved(void* x, const int64_t* positions, const float* freq, float mag, int64_t num_tokens,
                                     int heads, int rot_dim, int64_t token_stride, int64_t head_stride, int offset,
                                     int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && heads > 0 && rot_dim >= 0 && rot_dim % 2 == 0 && offset >= 0);
  if (num_tokens == 0 || rot_dim == 0) return SP_OK;
  SP_CHECK_ARG(x && positions && freq);
  SP_DISPATCH_DTYPE(dtype, (rotary_interleaved_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               x, positions, freq, mag, heads, rot_dim, token_stride, head_stride, offset)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_latent_kv_store(void* pool, int64_t pool_stride, const void* dkv, int64_t dkv_stride,
                                  const float* norm_w, const int64_t* positions, const float* freq, float mag,
                                  const int64_t* loc, int64_t num_tokens, int rank, int rot_dim, int rot_dims, float eps,
                                  int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && rank > 0 && rot_dim >= 0 && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(pool && dkv && norm_w && positions && loc && (freq || rot_dims == 0));
  SP_CHECK_ARG(pool_stride >= rank + rot_dim && dkv_stride >= rank + rot_dim);
  SP_DISPATCH_DTYPE(dtype, (latent_kv_store_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               pool, pool_stride, dkv, dkv_stride, norm_w, positions, freq, mag, loc, rank, rot_dim, rot_dims, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_latent_attention(void* out, const void* q_lat, const void* q_rot, const void* pool, int64_t pool_stride,
                                   const int32_t* req_to_token, int64_t table_stride, int64_t num_tokens, int heads,
                                   int rank, int rot_dim, int64_t qrot_token_stride, int64_t qrot_head_stride,
                                   float scale, SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && heads > 0 && rank > 0 && rot_dim >= 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && q_lat && pool && req_to_token && req_pool_indices && seq_lens && (q_rot || rot_dim == 0));
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SP_CHECK_ARG(pool_stride >= rank + rot_dim);
  if (rank > 64 * kMaxPerLane) return SP_ERR_UNSUPPORTED;
  const size_t lds = 4 * (size_t)(rank + rot_dim + 64) * sizeof(float);
  if (lds > 64 * 1024) return SP_ERR_UNSUPPORTED;
  SEQ_BATCH(s);
  const dim3 grid((unsigned)num_tokens, (unsigned)((heads + 3) / 4));
  SP_DISPATCH_DTYPE(dtype, (latent_attention_kernel<Tag><<<grid, 256, lds, (hipStream_t)stream>>>(
                               out, q_lat, q_rot, pool, pool_stride, req_to_token, table_stride, s, num_tokens, heads,
                               rank, rot_dim, qrot_token_stride, qrot_head_stride, scale)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}
