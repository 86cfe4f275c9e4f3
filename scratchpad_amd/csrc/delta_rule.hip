// Generalized delta rule: a per-head matrix state with a per-channel decay and a per-channel removal along the unit key.
// Per head, with r, k, v of a token, decay w and removal rate a per key channel, all of the recurrence in fp32:
//   u  = k / sqrt(|k|^2 + 1e-6)
//   S' = diag(w) S - (a * u) (u^T S) + k v^T            (both first terms read the state the previous token left)
//   o  = S'^T r
//   out = o / rms_head(o) * norm_w * sigmoid(g)
// The gates come from sp_delta_gates:
//   w = exp(-rate * sigmoid(W2 tanh(p) + w0))            (p = the low-rank projection's output)
//   a = sigmoid(apre + a_bias)
//
// One workgroup per (request, head): a column of S (one value channel) lives in the registers of 2, 4 or 8 neighbouring
// lanes; the request's tokens of this step are walked in order from the state the previous step left in the pool (zeros
// at a sequence's first token), staged through LDS in passes.  A token costs ONE sweep over the column: the update, the
// numerator and - on the state just completed - the next token's u^T S, then two independent sums over the column's lanes
// (register moves); no workgroup barrier.  Prompt portions and single decoded
// tokens take the same path, and the order of every sum depends on the head only.
#include "seq_batch.h"

namespace sp {
namespace {

// w2t: [rank, channels] fp32 (the up-projection transposed: neighbouring threads read neighbouring channels).  A workgroup
// takes TPB tokens x 256 channels, a thread one channel: every weight it loads serves all TPB tokens (TPB = 8 for prompts'
// portions), and a step of few tokens (TPB = 1) still spreads over channels / 256 workgroups per token.
template <typename Tag, int TPB>
__global__ void __launch_bounds__(kBlock)
delta_gates_kernel(float* decay, float* remove, const void* p, int64_t p_stride, const float* w2t, const float* w0,
                   const void* apre, int64_t a_stride, const float* a_bias, int64_t T, int channels, int rank, float rate) {
  typedef Elem<Tag> E;
  extern __shared__ float tp[];                          // [TPB][rank]
  const int64_t t0 = (int64_t)blockIdx.x * TPB;
  const int c = blockIdx.y * kBlock + threadIdx.x;
  for (int e = threadIdx.x; e < TPB * rank; e += kBlock) {
    const int tt = e / rank, r = e % rank;
    tp[e] = t0 + tt < T ? tanhf(E::load(p, (t0 + tt) * p_stride + r)) : 0.f;
  }
  __syncthreads();
  if (c >= channels) return;
  float acc[TPB];
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) acc[tt] = 0.f;
  int r = 0;
  for (; r + 4 <= rank; r += 4) {                        // four weights in flight
    const float w_0 = w2t[(int64_t)r * channels + c], w_1 = w2t[(int64_t)(r + 1) * channels + c];
    const float w_2 = w2t[(int64_t)(r + 2) * channels + c], w_3 = w2t[(int64_t)(r + 3) * channels + c];
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt) {
      const float* q = tp + tt * rank + r;
      acc[tt] += w_0 * q[0];
      acc[tt] += w_1 * q[1];
      acc[tt] += w_2 * q[2];
      acc[tt] += w_3 * q[3];
    }
  }
  for (; r < rank; ++r) {
    const float w = w2t[(int64_t)r * channels + c];
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt) acc[tt] += w * tp[tt * rank + r];
  }
  const float bias = w0[c], ab = a_bias[c];
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) {
    const int64_t t = t0 + tt;
    if (t < T) {
      decay[t * channels + c] = expf(-rate / (1.f + expf(-(acc[tt] + bias))));
      remove[t * channels + c] = 1.f / (1.f + expf(-(E::load(apre, t * a_stride + c) + ab)));
    }
  }
}

constexpr int delta_chunk(int KP) { return KP > 64 ? 8 : 16; }                      // tokens staged in LDS per pass
// lanes that share one column of S: 8 state values per lane where the workgroup's 1024 threads allow it (measured at heads of
// 64: 2 lanes 1.07 ms, 4 lanes 0.58 ms, 8 lanes 0.38 ms, 16 lanes 0.49 ms per 4096 tokens with two sweeps per token and
// lane exchanges through LDS; 8 lanes 0.29 ms, 16 lanes 0.32 ms with one sweep and register moves - more waves per SIMD
// hide the waits of the per-token chain until the sums over the lanes take over)
constexpr int delta_split(int KP) { return KP > 128 ? 4 : (KP > 32 ? 8 : (KP > 16 ? 4 : 2)); }

// thread = (column col of S, part): part p of SP owns the rows [p DS, (p + 1) DS) of the column.  LDS rows are padded by
// 4 floats per part so that the parts' simultaneous broadcast reads fall into different banks.
// A pass's operands come from global memory into registers in ONE burst (every load issued before the first is used), and
// the burst of pass n + 1 is issued right before the token loop of pass n, so it flies while the recurrence runs; the loop
// itself touches LDS and registers only.
template <typename Tag, int KP>
__global__ void __launch_bounds__(KP * delta_split(KP) < 64 ? 64 : KP * delta_split(KP))
delta_recurrence_kernel(void* out, int64_t out_stride, const void* r, int64_t r_stride, const void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* decay,
                        const float* remove, const float* norm_w, float* state, int64_t state_stride, SeqBatch s, int H,
                        int K, float eps) {
  typedef Elem<Tag> E;
  constexpr int kChunk = delta_chunk(KP), SP = delta_split(KP), DS = KP / SP, ROW = KP + 4 * SP;
  constexpr int NT = KP * SP < 64 ? 64 : KP * SP;       // threads of the workgroup (the launch uses exactly these)
  constexpr int TSTEP = NT / KP, PER = kChunk / TSTEP;  // staging: thread j takes channel j % KP of tokens j / KP + u TSTEP
  constexpr int PERG = kChunk / SP;                     // epilogue: thread (col, part) takes tokens part + u SP
  // (rows and parts start at multiples of 16 bytes: the token loop reads them four floats at a time)
  __shared__ __attribute__((aligned(16))) float sr[kChunk][ROW], sk[kChunk][ROW], sw[kChunk][ROW], su[kChunk + 1][ROW], sau[kChunk][ROW];
  __shared__ float sv[kChunk][KP], so[kChunk][KP], sinv[kChunk];
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int wave = j >> 6, lane = j & 63, waves = NT >> 6;
  const int col = j / SP, part = j % SP;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = col < K;
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride + (int64_t)h * K * K;
  const bool held = prefix > 0;
  const int64_t hc = (int64_t)h * K, HK = (int64_t)H * K;
  const int mine = part * (DS + 4);
  const int si = j % KP, st0 = j / KP;                  // this thread's staged channel and first staged token
  const bool sok = si < K;
  const int sat = si + 4 * (si / DS);
  float fr[PER], fk[PER], fw[PER], fa[PER], fv[PER], fg[PERG];
  // the operands of the pass that starts at c0 (rows past the pass's end repeat its last row; they are never used)
  auto fetch = [&](int64_t c0) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int tt = st0 + u * TSTEP;
      const int64_t row = start + c0 + (tt < n ? tt : n - 1);
      fr[u] = sok ? E::load(r, row * r_stride + hc + si) : 0.f;
      fk[u] = sok ? E::load(k, row * k_stride + hc + si) : 0.f;
      fv[u] = sok ? E::load(v, row * v_stride + hc + si) : 0.f;
      fw[u] = sok ? decay[row * HK + hc + si] : 0.f;
      fa[u] = sok ? remove[row * HK + hc + si] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < PERG; ++u) {
      const int tt = part + u * SP;
      fg[u] = live ? E::load(g, (start + c0 + (tt < n ? tt : n - 1)) * g_stride + hc + col) : 0.f;
    }
  };
  fetch(0);
  float S[DS];
#pragma unroll
  for (int ii = 0; ii < DS; ++ii) {
    const int i = part * DS + ii;
    S[ii] = (live && i < K && held) ? st[(int64_t)i * K + col] : 0.f;
  }
  const float nw = live ? norm_w[hc + col] : 0.f;
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();                                     // the previous pass's epilogue is done with so and sinv
    float gate[PERG];
#pragma unroll
    for (int u = 0; u < PERG; ++u) gate[u] = fg[u];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int tt = st0 + u * TSTEP;
      sr[tt][sat] = fr[u];
      sk[tt][sat] = fk[u];
      sw[tt][sat] = fw[u];
      sau[tt][sat] = fa[u];
      sv[tt][si] = fv[u];
    }
    __syncthreads();
    // the unit key of every token of the pass: a wave per token
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < K; i += 64) {
        const float x = sk[tt][i + 4 * (i / DS)];
        ss += x * x;
      }
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss + 1e-6f);
      for (int i = lane; i < KP; i += 64) {
        const int at = i + 4 * (i / DS);
        const float uu = sk[tt][at] * inv;
        su[tt][at] = uu;
        sau[tt][at] *= uu;
      }
    }
    __syncthreads();
    if (c0 + kChunk < len) fetch(c0 + kChunk);           // in flight while the recurrence runs
    // u^T S of the pass's first token; every later token's is formed in the sweep that completes the state it reads
    // (four partial sums per sum: the chain of dependent additions is a quarter as long; DS is a multiple of 4)
    float proj;
    {
      const float4* pu = reinterpret_cast<const float4*>(&su[0][mine]);
      float pj[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DS; ii += 4) {
        const float4 u4 = pu[ii / 4];
        pj[0] += u4.x * S[ii];
        pj[1] += u4.y * S[ii + 1];
        pj[2] += u4.z * S[ii + 2];
        pj[3] += u4.w * S[ii + 3];
      }
      proj = lanes_sum<SP>((pj[0] + pj[1]) + (pj[2] + pj[3]));
    }
    for (int tt = 0; tt < n; ++tt) {
      const float4* pau = reinterpret_cast<const float4*>(&sau[tt][mine]);
      const float4* pw = reinterpret_cast<const float4*>(&sw[tt][mine]);
      const float4* pk = reinterpret_cast<const float4*>(&sk[tt][mine]);
      const float4* pr = reinterpret_cast<const float4*>(&sr[tt][mine]);
      const float4* pun = reinterpret_cast<const float4*>(&su[tt + 1][mine]);      // the next token's unit key (row n: unused)
      const float vj = live ? sv[tt][col] : 0.f;
      float nm[4] = {0.f, 0.f, 0.f, 0.f}, pj[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DS; ii += 4) {
        const float4 w4 = pw[ii / 4], a4 = pau[ii / 4], k4 = pk[ii / 4], r4 = pr[ii / 4], u4 = pun[ii / 4];
        S[ii] = w4.x * S[ii] - a4.x * proj + k4.x * vj;
        S[ii + 1] = w4.y * S[ii + 1] - a4.y * proj + k4.y * vj;
        S[ii + 2] = w4.z * S[ii + 2] - a4.z * proj + k4.z * vj;
        S[ii + 3] = w4.w * S[ii + 3] - a4.w * proj + k4.w * vj;
        nm[0] += S[ii] * r4.x;
        nm[1] += S[ii + 1] * r4.y;
        nm[2] += S[ii + 2] * r4.z;
        nm[3] += S[ii + 3] * r4.w;
        pj[0] += S[ii] * u4.x;
        pj[1] += S[ii + 1] * u4.y;
        pj[2] += S[ii + 2] * u4.z;
        pj[3] += S[ii + 3] * u4.w;
      }
      const float num = lanes_sum<SP>((nm[0] + nm[1]) + (nm[2] + nm[3]));
      proj = lanes_sum<SP>((pj[0] + pj[1]) + (pj[2] + pj[3]));
      if (live && part == 0) so[tt][col] = num;
    }
    __syncthreads();
    // per-head RMS of o, output weight and gate
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < K; i += 64) ss += so[tt][i] * so[tt][i];
      ss = wave_sum(ss);
      if (lane == 0) sinv[tt] = 1.f / sqrtf(ss / (float)K + eps);
    }
    __syncthreads();
    if (live) {
#pragma unroll
      for (int u = 0; u < PERG; ++u) {
        const int tt = part + u * SP;
        if (tt < n)
          E::store(out, (start + c0 + tt) * out_stride + hc + col, so[tt][col] * sinv[tt] * nw / (1.f + expf(-gate[u])));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < DS; ++ii) {
      const int i = part * DS + ii;
      if (i < K) st[(int64_t)i * K + col] = S[ii];
    }
  }
}

template <typename Tag>
static int launch_delta(void* out, int64_t out_stride, const void* r, int64_t r_stride, const void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, const void* g, int64_t g_stride, const float* decay,
                        const float* remove, const float* norm_w, float* state, int64_t state_stride, const SeqBatch& s,
                        int H, int K, float eps, hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
#define SP_DELTA(KP)                                                                                                    \
  delta_recurrence_kernel<Tag, KP><<<grid, (unsigned)(KP * delta_split(KP) < 64 ? 64 : KP * delta_split(KP)), 0, st>>>(  \
      out, out_stride, r, r_stride, k, k_stride, v, v_stride, g, g_stride, decay, remove, norm_w, state, state_stride, s, H, K, \
      eps)
  if (K <= 16) SP_DELTA(16);
  else if (K <= 32) SP_DELTA(32);
  else if (K <= 64) SP_DELTA(64);
  else if (K <= 128) SP_DELTA(128);
  else if (K <= 256) SP_DELTA(256);
  else return SP_ERR_UNSUPPORTED;
#undef SP_DELTA
  SP_LAUNCH_CHECK();
  return SP_OK;
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_delta_gates(float* decay, float* remove, const void* p, int64_t p_stride, const float* w2t, const float* w0,
                              const void* apre, int64_t a_stride, const float* a_bias, int64_t num_tokens, int channels,
                              int rank, float rate, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && channels > 0 && rank > 0 && rank <= 8192);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(decay && remove && p && w2t && w0 && apre && a_bias && p_stride >= rank && a_stride >= channels);
  const unsigned cb = (unsigned)((channels + kBlock - 1) / kBlock);
  if (num_tokens >= 64 && rank <= 1024) {
    SP_DISPATCH_DTYPE(dtype, (delta_gates_kernel<Tag, 8><<<dim3((unsigned)((num_tokens + 7) / 8), cb), kBlock,
                                                            8 * rank * sizeof(float), (hipStream_t)stream>>>(
                                 decay, remove, p, p_stride, w2t, w0, apre, a_stride, a_bias, num_tokens, channels, rank, rate)));
  } else {
    SP_DISPATCH_DTYPE(dtype, (delta_gates_kernel<Tag, 1><<<dim3((unsigned)num_tokens, cb), kBlock, rank * sizeof(float),
                                                            (hipStream_t)stream>>>(
                                 decay, remove, p, p_stride, w2t, w0, apre, a_stride, a_bias, num_tokens, channels, rank, rate)));
  }
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_delta_recurrence(void* out, int64_t out_stride, const void* r, int64_t r_stride, const void* k,
                                   int64_t k_stride, const void* v, int64_t v_stride, const void* g, int64_t g_stride,
                                   const float* decay, const float* remove, const float* norm_w, float* state,
                                   int64_t state_stride, int heads, int head_dim, float eps, SP_SEQ_PARAMS, int dtype,
                                   void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && head_dim > 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(out && r && k && v && g && decay && remove && norm_w && state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SP_CHECK_ARG(state_stride >= (int64_t)heads * head_dim * head_dim);
  const int64_t n = (int64_t)heads * head_dim;
  SP_CHECK_ARG(r_stride >= n && k_stride >= n && v_stride >= n && g_stride >= n && out_stride >= n);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_delta<Tag>(out, out_stride, r, r_stride, k, k_stride, v, v_stride, g, g_stride, decay,
                                                     remove, norm_w, state, state_stride, s, heads, head_dim, eps,
                                                     (hipStream_t)stream)));
}
