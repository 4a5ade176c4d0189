// State-space mixer (Mamba-2 form) and the small pieces recurrent mixers share.
//   gate projections   out[t, n] = bias[n] + sum_i w[n, i] x[t, i]        few outputs (one per head), fp32 weights,
//                                                                         fp32 accumulation and fp32 OUTPUT: what enters
//                                                                         a recurrence's decay or gate is never rounded
//   causal convolution out[t, c] = silu(bias[c] + sum_j w[c, j] in[t - (taps-1) + j, c])   per channel; inputs before a
//                      step's first row come from the request's saved last taps-1 inputs (zeros before the sequence)
//   scan               dt = softplus(dt_raw + dt_bias);  S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x
//                      per head, S [N, Dv] fp32 in the state pool; head h reads B, C of group h / (H / G)
//   gated group norm   out = (y silu(z)) / rms_part * w      the gate BEFORE the norm, `parts` equal parts per row
#include "seq_batch.h"

namespace sp {
namespace {

__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// one workgroup per (token, 16 outputs): every wave forms 4 outputs at once; a lane takes 4 neighbouring inputs per step
// (16-byte weight loads where rows allow) and several steps are in flight, so the loop does not wait load by load
template <typename Tag, bool VEC>
__global__ void __launch_bounds__(256)
small_linear_f32_kernel(float* out, const void* x, int64_t x_stride, const float* w, const float* bias, int64_t T, int K, int N) {
  typedef Elem<Tag> E;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  const int n0 = (blockIdx.y * 4 + wave) * 4;
  if (n0 >= N) return;
  // rows past N repeat the last row (computed, never stored): no branch in the loop
  const float* w0 = w + (int64_t)n0 * K;
  const float* w1 = w + (int64_t)(n0 + 1 < N ? n0 + 1 : N - 1) * K;
  const float* w2 = w + (int64_t)(n0 + 2 < N ? n0 + 2 : N - 1) * K;
  const float* w3 = w + (int64_t)(n0 + 3 < N ? n0 + 3 : N - 1) * K;
  float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
  if (VEC) {
#pragma unroll 4
    for (int i = 4 * lane; i < K; i += 256) {
      const u32x4 a0 = ld16(w0 + i), a1 = ld16(w1 + i), a2 = ld16(w2 + i), a3 = ld16(w3 + i);
      float xv[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) xv[e] = E::load(x, t * x_stride + i + e);
      d0 += as_f32(a0[0]) * xv[0] + as_f32(a0[1]) * xv[1] + as_f32(a0[2]) * xv[2] + as_f32(a0[3]) * xv[3];
      d1 += as_f32(a1[0]) * xv[0] + as_f32(a1[1]) * xv[1] + as_f32(a1[2]) * xv[2] + as_f32(a1[3]) * xv[3];
      d2 += as_f32(a2[0]) * xv[0] + as_f32(a2[1]) * xv[1] + as_f32(a2[2]) * xv[2] + as_f32(a2[3]) * xv[3];
      d3 += as_f32(a3[0]) * xv[0] + as_f32(a3[1]) * xv[1] + as_f32(a3[2]) * xv[2] + as_f32(a3[3]) * xv[3];
    }
  } else {
#pragma unroll 4
    for (int i = lane; i < K; i += 64) {
      const float xv = E::load(x, t * x_stride + i);
      d0 += w0[i] * xv;
      d1 += w1[i] * xv;
      d2 += w2[i] * xv;
      d3 += w3[i] * xv;
    }
  }
  d0 = wave_sum(d0), d1 = wave_sum(d1), d2 = wave_sum(d2), d3 = wave_sum(d3);
  if (lane == 0) {
    out[t * N + n0] = d0 + (bias ? bias[n0] : 0.f);
    if (n0 + 1 < N) out[t * N + n0 + 1] = d1 + (bias ? bias[n0 + 1] : 0.f);
    if (n0 + 2 < N) out[t * N + n0 + 2] = d2 + (bias ? bias[n0 + 2] : 0.f);
    if (n0 + 3 < N) out[t * N + n0 + 3] = d3 + (bias ? bias[n0 + 3] : 0.f);
  }
}

// state [slot][taps - 1][C]: entry k = the input at position (tokens held) - (taps - 1) + k
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
conv_silu_kernel(void* out, int64_t out_stride, const void* in, int64_t in_stride, const float* w, const float* bias,
                 const float* state, int64_t state_stride, SeqBatch s, int C, int taps) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * kBlock + threadIdx.x;
  if (c >= C) return;
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int64_t r = t - (taps - 1) + j;
    float val = 0.f;
    if (r >= start) {
      val = E::load(in, r * in_stride + c);
    } else {
      const int64_t back = start - r;                  // 1 .. taps - 1 rows before the step
      if (prefix - back >= 0) val = st[(int64_t)(taps - 1 - back) * C + c];
    }
    acc += w[(int64_t)c * taps + j] * val;
  }
  E::store(out, t * out_stride + c, acc / (1.f + expf(-acc)));
}

constexpr int kMaxTaps = 16;

template <typename Tag>
__global__ void __launch_bounds__(kBlock)
conv_state_kernel(float* state, int64_t state_stride, const void* in, int64_t in_stride, SeqBatch s, int C, int taps) {
  typedef Elem<Tag> E;
  const int b = blockIdx.x;
  const int c = blockIdx.y * kBlock + threadIdx.x;
  if (c >= C) return;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  const int keep = taps - 1;
  float fresh[kMaxTaps];
  for (int k = 0; k < keep; ++k) {
    const int64_t p = prefix + len - keep + k;       // position of the new entry k
    float val = 0.f;
    if (p >= prefix) val = E::load(in, (start + (p - prefix)) * in_stride + c);
    else if (p >= 0) val = st[(p - prefix + keep) * C + c];
    fresh[k] = val;
  }
  for (int k = 0; k < keep; ++k) st[(int64_t)k * C + c] = fresh[k];
}

constexpr int kChunk = 16;      // tokens staged in LDS per pass
// lanes that share one column of S: each holds at most 64 of the column's N values (at 128 per lane the state alone
// fills the register file, one wave per SIMD remains and every LDS read of B and C waits in full)
constexpr int split_of(int NP) { return NP > 64 ? 4 : (NP > 32 ? 2 : 1); }

// one workgroup per (request, head); thread = (column col of S, part): part p of SP owns the rows [p NS, (p + 1) NS) of
// the column, the parts are neighbouring lanes and add their partial outputs by lane exchange.  LDS rows of B and C are
// padded by 4 floats per part so that the parts' simultaneous broadcast reads fall into different banks.
template <typename Tag, int NP>
__global__ void __launch_bounds__(256 * split_of(NP))
mamba2_scan_kernel(float* y, int64_t y_stride, const void* xbc, int64_t xbc_stride, const float* dt_raw, const float* dt_bias,
                   const float* A_log, const float* Dskip, float* state, int64_t state_stride, SeqBatch s, int H, int G, int N,
                   int Dv) {
  typedef Elem<Tag> E;
  constexpr int SP = split_of(NP), NS = NP / SP, ROW = NP + 4 * SP;
  __shared__ float sB[kChunk][ROW], sC[kChunk][ROW], sdt[kChunk], sdec[kChunk];
  extern __shared__ float sx[];                         // [kChunk][Dv]: no global load inside the token loop
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int nthreads = blockDim.x;
  const int col = j / SP, part = j % SP;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = col < Dv;
  const int g = h / (H / G);
  const int64_t inner = (int64_t)H * Dv;
  const int64_t colx = (int64_t)h * Dv, colB = inner + (int64_t)g * N, colC = inner + (int64_t)G * N + (int64_t)g * N;
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride + (int64_t)h * N * Dv;
  float S[NS];
#pragma unroll
  for (int ii = 0; ii < NS; ++ii) {
    const int i = part * NS + ii;
    S[ii] = (live && i < N && prefix > 0) ? st[(int64_t)i * Dv + col] : 0.f;
  }
  const float a = expf(A_log[h]), bias = dt_bias[h], skip = Dskip[h];
  const float* myB = &sB[0][part * (NS + 4)];
  const float* myC = &sC[0][part * (NS + 4)];
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();
    // staging: every load of the pass is issued before the first is used (rows past the pass's end repeat its last row)
#pragma unroll
    for (int tt = 0; tt < kChunk; ++tt) {
      const int64_t row = start + c0 + (tt < n ? tt : n - 1);
      for (int i = j; i < NP; i += nthreads) {
        const bool ok = i < N;
        const int at = i + 4 * (i / NS);
        sB[tt][at] = ok ? E::load(xbc, row * xbc_stride + colB + i) : 0.f;
        sC[tt][at] = ok ? E::load(xbc, row * xbc_stride + colC + i) : 0.f;
      }
      for (int c = j; c < Dv; c += nthreads) sx[tt * Dv + c] = E::load(xbc, row * xbc_stride + colx + c);
    }
    if (j < n) {
      const float dt = softplus_f(dt_raw[(start + c0 + j) * H + h] + bias);
      sdt[j] = dt;
      sdec[j] = expf(-a * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const int64_t row = start + c0 + tt;
      const float xj = live ? sx[tt * Dv + col] : 0.f;
      const float dec = sdec[tt], dx = sdt[tt] * xj;
      const float* Bt = myB + tt * ROW;
      const float* Ct = myC + tt * ROW;
      float o = 0.f;
#pragma unroll
      for (int ii = 0; ii < NS; ++ii) {
        S[ii] = dec * S[ii] + Bt[ii] * dx;
        o += S[ii] * Ct[ii];
      }
#pragma unroll
      for (int off = 1; off < SP; off <<= 1) o += __shfl_xor(o, off, 64);
      if (live && part == 0) y[row * y_stride + colx + col] = o + skip * xj;
    }
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < NS; ++ii) {
      const int i = part * NS + ii;
      if (i < N) st[(int64_t)i * Dv + col] = S[ii];
    }
  }
}

template <typename Tag>
__global__ void __launch_bounds__(kBlock)
gated_group_norm_kernel(void* out, int64_t out_stride, const float* y, int64_t y_stride, const void* z, int64_t z_stride,
                        const float* w, int n, int parts, float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  const int per = n / parts;
  for (int p = 0; p < parts; ++p) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < per; i += blockDim.x) {
      const float zv = E::load(z, t * z_stride + p * per + i);
      const float v = y[t * y_stride + p * per + i] * (zv / (1.f + expf(-zv)));
      ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)per + eps);
    for (int i = threadIdx.x; i < per; i += blockDim.x) {
      const int c = p * per + i;
      const float zv = E::load(z, t * z_stride + c);
      E::store(out, t * out_stride + c, y[t * y_stride + c] * (zv / (1.f + expf(-zv))) * inv * w[c]);
    }
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_small_linear_f32(float* out, const void* x, int64_t x_stride, const float* weight, const float* bias,
                                   int64_t num_tokens, int k, int n, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && k > 0 && n > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && x && weight && x_stride >= k);
  const dim3 grid((unsigned)num_tokens, (unsigned)((n + 15) / 16));
  if (k % 4 == 0 && ((uintptr_t)weight & 15) == 0)
    SP_DISPATCH_DTYPE(dtype, (small_linear_f32_kernel<Tag, true><<<grid, 256, 0, (hipStream_t)stream>>>(
                                 out, x, x_stride, weight, bias, num_tokens, k, n)));
  else
    SP_DISPATCH_DTYPE(dtype, (small_linear_f32_kernel<Tag, false><<<grid, 256, 0, (hipStream_t)stream>>>(
                                 out, x, x_stride, weight, bias, num_tokens, k, n)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_causal_conv_silu(void* out, int64_t out_stride, const void* in, int64_t in_stride, const float* weight,
                                   const float* bias, float* state, int64_t state_stride, int64_t num_tokens, int channels,
                                   int taps, SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && channels > 0 && taps >= 1 && taps <= kMaxTaps);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && in && weight && req_pool_indices && seq_lens);
  SP_CHECK_ARG(out_stride >= channels && in_stride >= channels);
  SP_CHECK_ARG(taps == 1 || (state && state_stride >= (int64_t)(taps - 1) * channels));      // one tap: nothing is carried
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SEQ_BATCH(s);
  const unsigned cb = (unsigned)((channels + kBlock - 1) / kBlock);
  SP_DISPATCH_DTYPE(dtype, (conv_silu_kernel<Tag><<<dim3((unsigned)num_tokens, cb), kBlock, 0, (hipStream_t)stream>>>(
                               out, out_stride, in, in_stride, weight, bias, state, state_stride, s, channels, taps)));
  SP_LAUNCH_CHECK();
  if (taps > 1) {      // after every reader of the old state (stream order)
    SP_DISPATCH_DTYPE(dtype, (conv_state_kernel<Tag><<<dim3((unsigned)batch_size, cb), kBlock, 0, (hipStream_t)stream>>>(
                                 state, state_stride, in, in_stride, s, channels, taps)));
    SP_LAUNCH_CHECK();
  }
  return SP_OK;
}

template <typename Tag>
static int launch_mamba2(float* y, int64_t y_stride, const void* xbc, int64_t xbc_stride, const float* dt_raw,
                         const float* dt_bias, const float* A_log, const float* Dskip, float* state, int64_t state_stride,
                         const SeqBatch& s, int H, int G, int N, int Dv, hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
#define SP_SCAN(NP)                                                                                                    \
  mamba2_scan_kernel<Tag, NP><<<grid, (unsigned)((Dv * split_of(NP) + 63) / 64 * 64), (size_t)kChunk * Dv * sizeof(float), st>>>(y, y_stride, xbc, xbc_stride, dt_raw, dt_bias, A_log, Dskip, state, \
                                                        state_stride, s, H, G, N, Dv)
  if (N <= 16) SP_SCAN(16);
  else if (N <= 32) SP_SCAN(32);
  else if (N <= 64) SP_SCAN(64);
  else if (N <= 128) SP_SCAN(128);
  else if (N <= 256) SP_SCAN(256);
  else return SP_ERR_UNSUPPORTED;
#undef SP_SCAN
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_mamba2_scan(float* y, int64_t y_stride, const void* xbc, int64_t xbc_stride, const float* dt_raw,
                              const float* dt_bias, const float* A_log, const float* Dskip, float* state,
                              int64_t state_stride, int heads, int groups, int state_size, int vdim, SP_SEQ_PARAMS,
                              int dtype, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && state_size > 0 && vdim > 0 && vdim <= 256);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(y && xbc && dt_raw && dt_bias && A_log && Dskip && state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  const int64_t inner = (int64_t)heads * vdim;
  SP_CHECK_ARG(y_stride >= inner && xbc_stride >= inner + 2 * (int64_t)groups * state_size);
  SP_CHECK_ARG(state_stride >= (int64_t)heads * state_size * vdim);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_mamba2<Tag>(y, y_stride, xbc, xbc_stride, dt_raw, dt_bias, A_log, Dskip, state,
                                                      state_stride, s, heads, groups, state_size, vdim, (hipStream_t)stream)));
}

extern "C" int sp_gated_group_norm(void* out, int64_t out_stride, const float* y, int64_t y_stride, const void* z,
                                   int64_t z_stride, const float* weight, int64_t num_tokens, int n, int parts, float eps,
                                   int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && n > 0 && parts > 0 && n % parts == 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && y && z && weight && out_stride >= n && y_stride >= n && z_stride >= n);
  SP_DISPATCH_DTYPE(dtype, (gated_group_norm_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               out, out_stride, y, y_stride, z, z_stride, weight, n, parts, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}
