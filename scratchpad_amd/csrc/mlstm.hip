// Matrix-memory recurrence with exponential gating kept stable by a running maximum (the mLSTM cell of xLSTM).
// Per head, with log gates i and f of a token and state (S [D, Dv], n [D], m), all fp32:
//   i = cap tanh(ipre / cap)                 f = logsigmoid(cap tanh(fpre / cap))         (ipre, fpre: fp32 projections)
//   m' = max(f + m, i)
//   S' = exp(f + m - m') S + exp(i - m') k v^T          n' = exp(f + m - m') n + exp(i - m') k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)      q = (projection) * D^(-1/2)
//   out = o / rms_head(o) * w * sigmoid(g)
// S, n and m start at ZERO for a sequence (m too: not minus infinity).  One workgroup per (request, head): thread j owns
// column j of S in registers; every wave keeps its own copy of n in LDS (all copies identical), so a token costs no
// workgroup barrier; tokens are staged through LDS in passes and the per-head norm and gate run as the pass's epilogue.
#include "seq_batch.h"

namespace sp {
namespace {

constexpr int kChunk = 8;

__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename Tag, int DP>
__global__ void __launch_bounds__(256)
mlstm_scan_kernel(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                  const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* ipre, const float* fpre,
                  const float* norm_w, float* S_state, int64_t S_stride, float* n_state, int64_t n_stride, float* m_state,
                  int64_t m_stride, SeqBatch s, int H, int D, int Dv, float cap, float eps) {
  typedef Elem<Tag> E;
  __shared__ float sq[kChunk][DP], sk[kChunk][DP], si[kChunk], sf[kChunk], sn[4][DP];
  extern __shared__ float so[];                         // [kChunk][Dv]
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int nthreads = blockDim.x, wave = j >> 6, lane = j & 63, waves = nthreads >> 6;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = j < Dv;
  const int64_t slot = load_idx(s.req_pool_indices, b, s.idx64);
  float* Sst = S_state + slot * S_stride + (int64_t)h * D * Dv;
  float* nst = n_state + slot * n_stride + (int64_t)h * D;
  float* mst = m_state + slot * m_stride + h;
  const bool held = prefix > 0;
  float S[DP];
#pragma unroll
  for (int i = 0; i < DP; ++i) S[i] = (live && i < D && held) ? Sst[(int64_t)i * Dv + j] : 0.f;
  for (int i = lane; i < DP; i += 64) sn[wave][i] = (i < D && held) ? nst[i] : 0.f;
  float m = held ? mst[0] : 0.f;
  const float qscale = 1.f / sqrtf((float)D);
  const int64_t colk = (int64_t)h * D, colv = (int64_t)h * Dv;
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();
    for (int e = j; e < n * DP; e += nthreads) {
      const int tt = e / DP, i = e % DP;
      const int64_t row = start + c0 + tt;
      const bool ok = i < D;
      sq[tt][i] = ok ? E::load(q, row * q_stride + colk + i) * qscale : 0.f;
      sk[tt][i] = ok ? E::load(k, row * k_stride + colk + i) : 0.f;
    }
    if (j < n) {
      const int64_t row = start + c0 + j;
      si[j] = cap * tanhf(ipre[row * H + h] / cap);
      sf[j] = logsigmoid_f(cap * tanhf(fpre[row * H + h] / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const int64_t row = start + c0 + tt;
      const float ig = si[tt], fg = sf[tt];
      const float m_new = fmaxf(fg + m, ig);
      const float keep = expf(fg + m - m_new), take = expf(ig - m_new);
      m = m_new;
      // this wave's copy of n, then n . q
      float part = 0.f;
      for (int i = lane; i < DP; i += 64) {
        const float nv = keep * sn[wave][i] + take * sk[tt][i];
        sn[wave][i] = nv;
        part += nv * sq[tt][i];
      }
      const float dot = wave_sum(part);
      const float tv = take * (live ? E::load(v, row * v_stride + colv + j) : 0.f);
      float num = 0.f;
#pragma unroll
      for (int i = 0; i < DP; ++i) {
        S[i] = keep * S[i] + sk[tt][i] * tv;
        num += S[i] * sq[tt][i];
      }
      if (live) so[tt * Dv + j] = num / (fmaxf(fabsf(dot), expf(-m_new)) + 1e-6f);
    }
    __syncthreads();
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < Dv; i += 64) ss += so[tt * Dv + i] * so[tt * Dv + i];
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
      const int64_t row = start + c0 + tt;
      for (int i = lane; i < Dv; i += 64) {
        const float gv = E::load(g, row * g_stride + colv + i);
        E::store(out, row * out_stride + colv + i, so[tt * Dv + i] * inv * norm_w[colv + i] / (1.f + expf(-gv)));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DP; ++i)
      if (i < D) Sst[(int64_t)i * Dv + j] = S[i];
  }
  if (wave == 0) {
    for (int i = lane; i < D; i += 64) nst[i] = sn[0][i];
    if (lane == 0) mst[0] = m;
  }
}

template <typename Tag>
static int launch_mlstm(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* ipre, const float* fpre,
                        const float* norm_w, float* S_state, int64_t S_stride, float* n_state, int64_t n_stride,
                        float* m_state, int64_t m_stride, const SeqBatch& s, int H, int D, int Dv, float cap, float eps,
                        hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
  const unsigned threads = (unsigned)((Dv + 63) / 64 * 64);
  const size_t lds = (size_t)kChunk * Dv * sizeof(float);
#define SP_MLSTM(DP)                                                                                                    \
  mlstm_scan_kernel<Tag, DP><<<grid, threads, lds, st>>>(out, out_stride, q, q_stride, k, k_stride, v, v_stride, g, g_stride, \
                                                         ipre, fpre, norm_w, S_state, S_stride, n_state, n_stride, m_state,  \
                                                         m_stride, s, H, D, Dv, cap, eps)
  if (D <= 16) SP_MLSTM(16);
  else if (D <= 32) SP_MLSTM(32);
  else if (D <= 64) SP_MLSTM(64);
  else if (D <= 128) SP_MLSTM(128);
  else if (D <= 256) SP_MLSTM(256);
  else return SP_ERR_UNSUPPORTED;
#undef SP_MLSTM
  SP_LAUNCH_CHECK();
  return SP_OK;
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_mlstm_scan(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                             const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* ipre,
                             const float* fpre, const float* norm_w, float* S_state, int64_t S_stride, float* n_state,
                             int64_t n_stride, float* m_state, int64_t m_stride, int heads, int dim, int vdim, float cap,
                             float eps, SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && dim > 0 && vdim > 0 && vdim <= 256 && cap > 0.f);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(out && q && k && v && g && ipre && fpre && norm_w && S_state && n_state && m_state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  const int64_t nk = (int64_t)heads * dim, nv = (int64_t)heads * vdim;
  SP_CHECK_ARG(q_stride >= nk && k_stride >= nk && v_stride >= nv && g_stride >= nv && out_stride >= nv);
  SP_CHECK_ARG(S_stride >= nk * vdim && n_stride >= nk && m_stride >= heads);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_mlstm<Tag>(out, out_stride, q, q_stride, k, k_stride, v, v_stride, g, g_stride, ipre,
                                                     fpre, norm_w, S_state, S_stride, n_state, n_stride, m_state, m_stride, s,
                                                     heads, dim, vdim, cap, eps, (hipStream_t)stream)));
}
