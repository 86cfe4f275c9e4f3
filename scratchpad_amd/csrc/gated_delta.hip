// Channel-gated delta rule: a per-head matrix state S [D, Dv] whose rows (key channels) each have a decay of their own,
// corrected along the unit key.  Per value head h (its query/key head is h / (H / G)), all of the recurrence in fp32:
//   qn = q / sqrt(|q|^2 + 1e-6) * D^(-1/2)       kn = k / sqrt(|k|^2 + 1e-6)        beta = sigmoid(bpre)
//   S  = diag(w) S                                (w: the token's decay per key channel)
//   u  = beta (v - S^T kn)                        (what the state does not yet return for this key)
//   S  = S + kn u^T                               o = S^T qn       (the read-out sees the token's own write)
//   out = o / rms_head(o) * norm_w * gate         (norm_w [Dv] shared by the heads, gate fp32 per value channel)
// Decay and gate come from sp_lowrank_gate, an fp32 product with a low-rank projection's output p [T, rank]:
//   z = W2 p + bias;   decay = exp(-exp(A_log[head]) softplus(z))   or   gate = sigmoid(z).
//
// One workgroup per (request, value head): a column of S (one value channel) lives in the registers of SP neighbouring
// lanes; the request's tokens of this step are walked in order from the state the previous step left in the pool (zeros at
// a sequence's first token), staged through LDS in passes.  A token costs ONE sweep over the column: the update, the
// read-out and - on the state just completed - the next token's (w * kn)^T S, then two independent sums over the column's
// lanes (register moves); no workgroup barrier inside a pass.  Prompt portions and single decoded tokens take the same
// path, and the order of every sum depends on the head's sizes only.
#include "seq_batch.h"

namespace sp {
namespace {

__device__ __forceinline__ float softplus_gd(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// w2t: [rank, channels] fp32 (the up-projection transposed: neighbouring threads read neighbouring channels).  A workgroup
// takes TPB tokens x 256 channels, a thread one channel: every weight it loads serves all TPB tokens.
// ACT 0: exp(-exp(A_log[c / per_head]) softplus(z));  ACT 1: sigmoid(z)
template <typename Tag, int TPB, int ACT>
__global__ void __launch_bounds__(kBlock)
lowrank_gate_kernel(float* out, const void* p, int64_t p_stride, const float* w2t, const float* bias, const float* A_log,
                    int64_t T, int channels, int rank, int per_head) {
  typedef Elem<Tag> E;
  extern __shared__ float tp[];                          // [TPB][rank]
  const int64_t t0 = (int64_t)blockIdx.x * TPB;
  const int c = blockIdx.y * kBlock + threadIdx.x;
  for (int e = threadIdx.x; e < TPB * rank; e += kBlock) {
    const int tt = e / rank, r = e % rank;
    tp[e] = t0 + tt < T ? E::load(p, (t0 + tt) * p_stride + r) : 0.f;
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
  const float b = bias ? bias[c] : 0.f;
  const float rate = ACT == 0 ? expf(A_log[c / per_head]) : 0.f;
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) {
    const int64_t t = t0 + tt;
    if (t < T) {
      const float z = acc[tt] + b;
      out[t * channels + c] = ACT == 0 ? expf(-rate * softplus_gd(z)) : 1.f / (1.f + expf(-z));
    }
  }
}

constexpr int gd_chunk(int KP) { return KP > 64 ? 8 : 16; }       // tokens staged in LDS per pass
constexpr int kGdMaxV = 256;                                      // value channels per head

// thread = (column col of S, part): part p of SP owns the rows [p DS, (p + 1) DS) of the column (DS = KP / SP, KP = the
// key width rounded up).  LDS rows are padded by 4 floats per part so that the parts' simultaneous broadcast reads fall
// into different banks.  The workgroup has ceil(Dv SP / 64) waves.
template <typename Tag, int KP, int SP>
__global__ void __launch_bounds__(1024)
gated_delta_scan_kernel(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, const void* bpre, int64_t b_stride, const float* decay,
                        const float* gate, const float* norm_w, float* state, int64_t state_stride, SeqBatch s, int H, int G,
                        int K, int Dv, float eps) {
  typedef Elem<Tag> E;
  constexpr int kChunk = gd_chunk(KP), DS = KP / SP, ROW = KP + 4 * SP;
  static_assert(DS % 4 == 0, "a part's rows are read four at a time");
  __shared__ __attribute__((aligned(16))) float sq[kChunk][ROW], sk[kChunk][ROW], sw[kChunk][ROW], sgk[kChunk + 1][ROW];
  __shared__ float sv[kChunk][kGdMaxV], so[kChunk][kGdMaxV], sbeta[kChunk], sinv[kChunk];
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x, NT = blockDim.x;
  const int wave = j >> 6, lane = j & 63, waves = NT >> 6;
  const int col = j / SP, part = j % SP;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = col < Dv;
  const int g = h / (H / G);
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride + (int64_t)h * K * Dv;
  const bool held = prefix > 0;
  const int64_t qc = (int64_t)g * K, wc = (int64_t)h * K, vc = (int64_t)h * Dv, HK = (int64_t)H * K, HV = (int64_t)H * Dv;
  const int mine = part * (DS + 4);
  const float qscale = 1.f / sqrtf((float)K);
  float S[DS];
#pragma unroll
  for (int ii = 0; ii < DS; ++ii) {
    const int i = part * DS + ii;
    S[ii] = (live && i < K && held) ? st[(int64_t)i * Dv + col] : 0.f;
  }
  const float nw = live ? norm_w[col] : 0.f;
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();                                     // the previous pass's epilogue is done with so and sinv
    for (int e = j; e < n * KP; e += NT) {
      const int tt = e / KP, i = e % KP;
      const int at = i + 4 * (i / DS);
      const int64_t row = start + c0 + tt;
      const bool ok = i < K;
      sq[tt][at] = ok ? E::load(q, row * q_stride + qc + i) : 0.f;
      sk[tt][at] = ok ? E::load(k, row * k_stride + qc + i) : 0.f;
      sw[tt][at] = ok ? decay[row * HK + wc + i] : 0.f;
    }
    for (int e = j; e < n * Dv; e += NT) {
      const int tt = e / Dv, i = e % Dv;
      sv[tt][i] = E::load(v, (start + c0 + tt) * v_stride + vc + i);
    }
    if (j < n) sbeta[j] = 1.f / (1.f + expf(-E::load(bpre, (start + c0 + j) * b_stride + h)));
    __syncthreads();
    // unit query and key of every token of the pass, and the decayed key: a wave per token
    for (int tt = wave; tt < n; tt += waves) {
      float sk2 = 0.f, sq2 = 0.f;
      for (int i = lane; i < K; i += 64) {
        const int at = i + 4 * (i / DS);
        sk2 += sk[tt][at] * sk[tt][at];
        sq2 += sq[tt][at] * sq[tt][at];
      }
      sk2 = wave_sum(sk2);
      sq2 = wave_sum(sq2);
      const float ik = 1.f / sqrtf(sk2 + 1e-6f), iq = qscale / sqrtf(sq2 + 1e-6f);
      for (int i = lane; i < KP; i += 64) {
        const int at = i + 4 * (i / DS);
        const float kn = sk[tt][at] * ik;
        sk[tt][at] = kn;
        sq[tt][at] *= iq;
        sgk[tt][at] = kn * sw[tt][at];
      }
    }
    __syncthreads();
    // (w * kn)^T S of the pass's first token; every later token's is formed in the sweep that completes the state it reads
    float proj;
    {
      const float4* pu = reinterpret_cast<const float4*>(&sgk[0][mine]);
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
      const float4* pw = reinterpret_cast<const float4*>(&sw[tt][mine]);
      const float4* pk = reinterpret_cast<const float4*>(&sk[tt][mine]);
      const float4* pq = reinterpret_cast<const float4*>(&sq[tt][mine]);
      const float4* pun = reinterpret_cast<const float4*>(&sgk[tt + 1][mine]);     // the next token's (row n: unused)
      const float u = live ? sbeta[tt] * (sv[tt][col] - proj) : 0.f;
      float nm[4] = {0.f, 0.f, 0.f, 0.f}, pj[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DS; ii += 4) {
        const float4 w4 = pw[ii / 4], k4 = pk[ii / 4], q4 = pq[ii / 4], u4 = pun[ii / 4];
        S[ii] = w4.x * S[ii] + k4.x * u;
        S[ii + 1] = w4.y * S[ii + 1] + k4.y * u;
        S[ii + 2] = w4.z * S[ii + 2] + k4.z * u;
        S[ii + 3] = w4.w * S[ii + 3] + k4.w * u;
        nm[0] += S[ii] * q4.x;
        nm[1] += S[ii + 1] * q4.y;
        nm[2] += S[ii + 2] * q4.z;
        nm[3] += S[ii + 3] * q4.w;
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
    // per-head RMS of o, then the output weight and gate
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < Dv; i += 64) ss += so[tt][i] * so[tt][i];
      ss = wave_sum(ss);
      if (lane == 0) sinv[tt] = 1.f / sqrtf(ss / (float)Dv + eps);
    }
    __syncthreads();
    for (int e = j; e < n * Dv; e += NT) {
      const int tt = e / Dv, i = e % Dv;
      const int64_t row = start + c0 + tt;
      E::store(out, row * out_stride + vc + i, so[tt][i] * sinv[tt] * norm_w[i] * gate[row * HV + vc + i]);
    }
  }
  (void)nw;
  if (live) {
#pragma unroll
    for (int ii = 0; ii < DS; ++ii) {
      const int i = part * DS + ii;
      if (i < K) st[(int64_t)i * Dv + col] = S[ii];
    }
  }
}

template <typename Tag>
static int launch_gated_delta(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                              const void* v, int64_t v_stride, const void* bpre, int64_t b_stride, const float* decay,
                              const float* gate, const float* norm_w, float* state, int64_t state_stride, const SeqBatch& s,
                              int H, int G, int K, int Dv, float eps, hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
#define SP_GD(KP, SPL)                                                                                                   \
  gated_delta_scan_kernel<Tag, KP, SPL><<<grid, (unsigned)((Dv * SPL + 63) / 64 * 64), 0, st>>>(                          \
      out, out_stride, q, q_stride, k, k_stride, v, v_stride, bpre, b_stride, decay, gate, norm_w, state, state_stride, s, H, \
      G, K, Dv, eps)
  // lanes per column: 8 state values per lane where the workgroup's 1024 threads allow it
  const bool wide = Dv > 128;                            // 8 lanes per column would need more than 1024 threads
  if (K <= 16) SP_GD(16, 2);
  else if (K <= 32) SP_GD(32, 4);
  else if (K <= 64) { if (wide) SP_GD(64, 4); else SP_GD(64, 8); }
  else if (K <= 128) { if (wide) SP_GD(128, 4); else SP_GD(128, 8); }
  else if (K <= 256) SP_GD(256, 4);
  else return SP_ERR_UNSUPPORTED;
#undef SP_GD
  SP_LAUNCH_CHECK();
  return SP_OK;
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_lowrank_gate(float* out, const void* p, int64_t p_stride, const float* w2t, const float* bias,
                               const float* A_log, int64_t num_tokens, int channels, int rank, int per_head, int act,
                               int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && channels > 0 && rank > 0 && rank <= 8192 && (act == 0 || act == 1));
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && p && w2t && p_stride >= rank);
  SP_CHECK_ARG(act != 0 || (A_log && per_head > 0 && channels % per_head == 0));
  const unsigned cb = (unsigned)((channels + kBlock - 1) / kBlock);
  if (per_head <= 0) per_head = 1;
#define SP_LG(TPB, ACT)                                                                                                  \
  SP_DISPATCH_DTYPE(dtype, (lowrank_gate_kernel<Tag, TPB, ACT><<<dim3((unsigned)((num_tokens + TPB - 1) / TPB), cb), kBlock, \
                                                                  TPB * rank * sizeof(float), (hipStream_t)stream>>>(     \
                               out, p, p_stride, w2t, bias, A_log, num_tokens, channels, rank, per_head)))
  if (num_tokens >= 64 && rank <= 1024) {
    if (act == 0) SP_LG(8, 0);
    else SP_LG(8, 1);
  } else {
    if (act == 0) SP_LG(1, 0);
    else SP_LG(1, 1);
  }
#undef SP_LG
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_gated_delta_scan(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k,
                                   int64_t k_stride, const void* v, int64_t v_stride, const void* bpre, int64_t b_stride,
                                   const float* decay, const float* gate, const float* norm_w, float* state,
                                   int64_t state_stride, int heads, int kv_heads, int dim, int vdim, float eps,
                                   SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(out && q && k && v && bpre && decay && gate && norm_w && state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SP_CHECK_ARG(state_stride >= (int64_t)heads * dim * vdim);
  SP_CHECK_ARG(q_stride >= (int64_t)kv_heads * dim && k_stride >= (int64_t)kv_heads * dim && b_stride >= heads);
  SP_CHECK_ARG(v_stride >= (int64_t)heads * vdim && out_stride >= (int64_t)heads * vdim);
  if (vdim > kGdMaxV) return SP_ERR_UNSUPPORTED;
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_gated_delta<Tag>(out, out_stride, q, q_stride, k, k_stride, v, v_stride, bpre, b_stride,
                                                           decay, gate, norm_w, state, state_stride, s, heads, kv_heads, dim,
                                                           vdim, eps, (hipStream_t)stream)));
}
