// Matrix-memory recurrence with exponential gating kept stable by a running maximum (the mLSTM cell of xLSTM).
// Per head, with log gates i and f of a token and state (S [D, Dv], n [D], m), all fp32:
//   i = cap tanh(ipre / cap)                 f = logsigmoid(cap tanh(fpre / cap))         (ipre, fpre: fp32 projections)
//   m' = max(f + m, i)
//   S' = exp(f + m - m') S + exp(i - m') k v^T          n' = exp(f + m - m') n + exp(i - m') k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)      q = (projection) * D^(-1/2)
//   out = o / rms_head(o) * w * sigmoid(g)
// S, n and m start at ZERO for a sequence (m too: not minus infinity).  One workgroup per (request, head): a column of S
// lives in the registers of 1, 2 or 4 neighbouring lanes and n is one more column, so a token costs no workgroup barrier
// and no sum over a wave; tokens are staged through LDS in passes and the per-head norm and gate run as the pass's epilogue.
#include "seq_batch.h"

namespace sp {
namespace {

// tokens staged in LDS per pass (fewer for the widest heads: static + dynamic LDS stay under 64 KB)
constexpr int chunk_of(int DP) { return DP > 128 ? 8 : 16; }
// lanes that share one column of S: each holds 16 - 64 of the column's D values, so the state never crowds the register
// file (at 128 values per lane the compiler is at its 256-register limit with one wave per SIMD) and a head gives the
// chip more waves - the recurrence is a chain of waits per token, and idle SIMDs are what a prompt leaves most of
constexpr int split_of(int DP) { return DP > 64 ? 4 : (DP > 32 ? 2 : 1); }

__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// thread = (column col of S, part): part p of SP owns the rows [p DS, (p + 1) DS) of the column; the parts of a column
// are neighbouring lanes and add their partial numerators by lane exchange.  LDS rows of q and k are padded by 4 floats
// per part so that the parts' simultaneous broadcast reads fall into different banks.
// The normaliser n is column Dv of the same recurrence (its "value" is 1): its lanes form n . q like any numerator, and
// the division by max(|n . q|, exp(-m)) + 1e-6 waits for the pass's epilogue - no sum over a wave inside the token loop.
template <typename Tag, int DP>
__global__ void __launch_bounds__(split_of(DP) == 1 ? 320 : (split_of(DP) == 2 ? 576 : 1024))
mlstm_scan_kernel(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                  const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* ipre, const float* fpre,
                  const float* norm_w, float* S_state, int64_t S_stride, float* n_state, int64_t n_stride, float* m_state,
                  int64_t m_stride, SeqBatch s, int H, int D, int Dv, float cap, float eps) {
  typedef Elem<Tag> E;
  constexpr int kChunk = chunk_of(DP), SP = split_of(DP), DS = DP / SP, ROW = DP + 4 * SP;
  __shared__ float sq[kChunk][ROW], sk[kChunk][ROW], si[kChunk], sf[kChunk], sinv[kChunk], sden[kChunk], sm[kChunk];
  extern __shared__ float so[];                         // [kChunk][Dv + 1] numerators (column Dv: n . q), then [kChunk][Dv] values
  float* sv = so + (size_t)kChunk * (Dv + 1);           // (no global load inside the token loop)
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int nthreads = blockDim.x, wave = j >> 6, lane = j & 63, waves = nthreads >> 6;
  const int col = j / SP, part = j % SP;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = col <= Dv, isn = col == Dv;         // column Dv is the normaliser
  const int64_t slot = load_idx(s.req_pool_indices, b, s.idx64);
  float* Sst = S_state + slot * S_stride + (int64_t)h * D * Dv;
  float* nst = n_state + slot * n_stride + (int64_t)h * D;
  float* mst = m_state + slot * m_stride + h;
  const bool held = prefix > 0;
  float S[DS];
#pragma unroll
  for (int ii = 0; ii < DS; ++ii) {
    const int i = part * DS + ii;
    S[ii] = (live && i < D && held) ? (isn ? nst[i] : Sst[(int64_t)i * Dv + col]) : 0.f;
  }
  float m = held ? mst[0] : 0.f;
  const float qscale = 1.f / sqrtf((float)D);
  const int64_t colk = (int64_t)h * D, colv = (int64_t)h * Dv;
  const float* myq = &sq[0][part * (DS + 4)];
  const float* myk = &sk[0][part * (DS + 4)];
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();
    // staging: every load of the pass is issued before the first is used (rows past the pass's end repeat its last row)
#pragma unroll
    for (int tt = 0; tt < kChunk; ++tt) {
      const int64_t row = start + c0 + (tt < n ? tt : n - 1);
      for (int i = j; i < DP; i += nthreads) {
        const bool ok = i < D;
        const int at = i + 4 * (i / DS);
        sq[tt][at] = ok ? E::load(q, row * q_stride + colk + i) * qscale : 0.f;
        sk[tt][at] = ok ? E::load(k, row * k_stride + colk + i) : 0.f;
      }
      for (int c = j; c < Dv; c += nthreads) sv[tt * Dv + c] = E::load(v, row * v_stride + colv + c);
    }
    if (j < n) {
      const int64_t row = start + c0 + j;
      si[j] = cap * tanhf(ipre[row * H + h] / cap);
      sf[j] = logsigmoid_f(cap * tanhf(fpre[row * H + h] / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float ig = si[tt], fg = sf[tt];
      const float m_new = fmaxf(fg + m, ig);
      const float keep = expf(fg + m - m_new), take = expf(ig - m_new);
      m = m_new;
      const float tv = take * (isn ? 1.f : (live ? sv[tt * Dv + col] : 0.f));
      const float* kq = myk + tt * ROW;
      const float* qq = myq + tt * ROW;
      float num = 0.f;
#pragma unroll
      for (int ii = 0; ii < DS; ++ii) {
        S[ii] = keep * S[ii] + kq[ii] * tv;
        num += S[ii] * qq[ii];
      }
#pragma unroll
      for (int off = 1; off < SP; off <<= 1) num += __shfl_xor(num, off, 64);
      if (live && part == 0) so[tt * (Dv + 1) + col] = num;
      if (j == 0) sm[tt] = m_new;
    }
    __syncthreads();
    // the division, then the per-head RMS of every token of the pass (a wave per token, LDS only), then every column of
    // all tokens at once
    for (int tt = wave; tt < n; tt += waves) {
      const float den = 1.f / (fmaxf(fabsf(so[tt * (Dv + 1) + Dv]), expf(-sm[tt])) + 1e-6f);
      float ss = 0.f;
      for (int i = lane; i < Dv; i += 64) {
        const float o = so[tt * (Dv + 1) + i] * den;
        ss += o * o;
      }
      ss = wave_sum(ss);
      if (lane == 0) {
        sden[tt] = den;
        sinv[tt] = 1.f / sqrtf(ss / (float)Dv + eps);
      }
    }
    __syncthreads();
    if (col < Dv) {                                     // part p takes the tokens p, p + SP, ...
      const float nw = norm_w[colv + col];
      constexpr int PER = kChunk / SP;
      float gv[PER];
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int tt = part + u * SP;
        gv[u] = E::load(g, (start + c0 + (tt < n ? tt : n - 1)) * g_stride + colv + col);
      }
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int tt = part + u * SP;
        if (tt < n)
          E::store(out, (start + c0 + tt) * out_stride + colv + col,
                   so[tt * (Dv + 1) + col] * sden[tt] * sinv[tt] * nw / (1.f + expf(-gv[u])));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < DS; ++ii) {
      const int i = part * DS + ii;
      if (i < D) {
        if (isn) nst[i] = S[ii];
        else Sst[(int64_t)i * Dv + col] = S[ii];
      }
    }
  }
  if (j == 0) mst[0] = m;
}

template <typename Tag>
static int launch_mlstm(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* ipre, const float* fpre,
                        const float* norm_w, float* S_state, int64_t S_stride, float* n_state, int64_t n_stride,
                        float* m_state, int64_t m_stride, const SeqBatch& s, int H, int D, int Dv, float cap, float eps,
                        hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
  if ((Dv + 1) * (D > 64 ? 4 : (D > 32 ? 2 : 1)) > 1024) return SP_ERR_UNSUPPORTED;      // vdim 256 with dim > 64
#define SP_MLSTM(DP)                                                                                                    \
  mlstm_scan_kernel<Tag, DP><<<grid, (unsigned)(((Dv + 1) * split_of(DP) + 63) / 64 * 64),                              \
                               (size_t)chunk_of(DP) * (2 * Dv + 1) * sizeof(float), st>>>(                              \
      out, out_stride, q, q_stride, k, k_stride, v, v_stride, g, g_stride, ipre, fpre, norm_w, S_state, S_stride, n_state,  \
      n_stride, m_state, m_stride, s, H, D, Dv, cap, eps)
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
