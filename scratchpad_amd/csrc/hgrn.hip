// Gated linear attention whose forget gate also decides what is written (the HGRN2 recurrence).
// Per head, with a query q [D], a value v [Dv] and a forget gate f [D] of a token, state S [D, Dv], all fp32:
//   q = silu(qpre)                f = lower + (1 - lower) * sigmoid(fpre + f_bias)
//   S' = diag(f) S + (1 - f) v^T          o = S'^T q
//   out = o / rms_head(o) * norm_w         (norm_w [Dv], the same for every head)
// There is no key: the row of S that belongs to query channel i takes in (1 - f_i) of the value.
//
// One workgroup per (request, head): a column of S (one value channel) lives in the registers of 1 to 8 neighbouring
// lanes; the request's tokens of this step are walked in order from the state the previous step left in the pool (zeros at
// a sequence's first token), staged through LDS in passes of 16 tokens, the head norm as the pass's epilogue.
#include "seq_batch.h"

namespace sp {
namespace {

constexpr int hgrn_chunk(int DP) { return DP > 128 ? 8 : 16; }
// lanes that share one column of S: 8 state values per lane (more waves per SIMD fill the waits of a wave's per-token chain)
// where the workgroup's 1024 threads hold vdim columns of that many lanes, else the coarser split that always fits
constexpr int hgrn_split_fine(int DP) { return DP / 8 > 8 ? 8 : DP / 8; }
constexpr int hgrn_split_coarse(int DP) { return DP > 64 ? 4 : (DP > 32 ? 2 : 1); }

// A pass's operands come from global memory into registers in ONE burst (every load issued before the first is used), and
// the burst of pass n + 1 is issued right before the token loop of pass n, so it flies while the recurrence runs; the loop
// itself touches LDS and registers only.  NT threads: Dv columns x SP parts, rounded up to whole waves.
template <typename Tag, int DP, int SP, int NT>
__global__ void __launch_bounds__(NT)
hgrn2_scan_kernel(void* out, int64_t out_stride, const void* qpre, int64_t q_stride, const void* fpre, int64_t f_stride,
                  const void* v, int64_t v_stride, const float* f_bias, const float* lower, const float* norm_w, float* state,
                  int64_t state_stride, SeqBatch s, int H, int D, int Dv, float eps) {
  typedef Elem<Tag> E;
  constexpr int kChunk = hgrn_chunk(DP), DS = DP / SP, ROW = DP + 4 * SP;
  constexpr int PERK = (kChunk * DP + NT - 1) / NT;     // staged (token, query channel) elements per thread and pass
  constexpr int PERV = kChunk / SP;                     // value / output tokens per thread: tokens part + u SP of column col
  // (rows and parts start at multiples of 16 bytes: the token loop reads them four floats at a time)
  __shared__ __attribute__((aligned(16))) float sq[kChunk][ROW], sf[kChunk][ROW];
  __shared__ float sinv[kChunk];
  extern __shared__ float so[];                         // [kChunk][Dv] numerators, then [kChunk][Dv] values
  float* sv = so + (size_t)kChunk * Dv;
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int wave = j >> 6, lane = j & 63, waves = NT >> 6;
  const int col = j / SP, part = j % SP;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const bool live = col < Dv;
  float* st = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride + (int64_t)h * D * Dv;
  const bool held = prefix > 0;
  const int64_t colk = (int64_t)h * D, colv = (int64_t)h * Dv;
  const int mine = part * (DS + 4);
  float fq[PERK], ff[PERK], fvv[PERV];
  // the operands of the pass that starts at c0 (rows past the pass's end repeat its last row; they are never used)
  auto fetch = [&](int64_t c0) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
#pragma unroll
    for (int u = 0; u < PERK; ++u) {
      const int e = j + u * NT, tt = e / DP, i = e % DP;
      const bool ok = e < kChunk * DP && i < D;
      const int64_t row = start + c0 + (tt < n ? tt : n - 1);
      fq[u] = ok ? E::load(qpre, row * q_stride + colk + i) : 0.f;
      ff[u] = ok ? E::load(fpre, row * f_stride + colk + i) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < PERV; ++u) {
      const int tt = part + u * SP;
      fvv[u] = live ? E::load(v, (start + c0 + (tt < n ? tt : n - 1)) * v_stride + colv + col) : 0.f;
    }
  };
  fetch(0);
  float S[DS];
#pragma unroll
  for (int ii = 0; ii < DS; ++ii) {
    const int i = part * DS + ii;
    S[ii] = (live && i < D && held) ? st[(int64_t)i * Dv + col] : 0.f;
  }
  // gate constants of this thread's staged channels (the same channel in every pass)
  float flo[PERK], fbi[PERK];
#pragma unroll
  for (int u = 0; u < PERK; ++u) {
    const int e = j + u * NT, i = e % DP;
    const bool ok = e < kChunk * DP && i < D;
    flo[u] = ok ? lower[colk + i] : 0.f;
    fbi[u] = ok ? f_bias[colk + i] : 0.f;
  }
  const float nw = live ? norm_w[col] : 0.f;
  for (int64_t c0 = 0; c0 < len; c0 += kChunk) {
    const int n = (int)(len - c0 < kChunk ? len - c0 : kChunk);
    __syncthreads();                                     // the previous pass's epilogue is done with so and sinv
#pragma unroll
    for (int u = 0; u < PERK; ++u) {
      const int e = j + u * NT, tt = e / DP, i = e % DP;
      if (e < kChunk * DP) {
        const int at = i + 4 * (i / DS);
        const bool ok = i < D;                           // register rows past D: f = 0 and q = 0, never stored
        sq[tt][at] = ok ? fq[u] / (1.f + expf(-fq[u])) : 0.f;
        sf[tt][at] = ok ? flo[u] + (1.f - flo[u]) / (1.f + expf(-(ff[u] + fbi[u]))) : 0.f;
      }
    }
    if (live) {
#pragma unroll
      for (int u = 0; u < PERV; ++u) sv[(part + u * SP) * Dv + col] = fvv[u];
    }
    __syncthreads();
    if (c0 + kChunk < len) fetch(c0 + kChunk);           // in flight while the recurrence runs
    for (int tt = 0; tt < n; ++tt) {
      const float4* pf = reinterpret_cast<const float4*>(&sf[tt][mine]);
      const float4* pq = reinterpret_cast<const float4*>(&sq[tt][mine]);
      const float vj = live ? sv[tt * Dv + col] : 0.f;
      float nm[4] = {0.f, 0.f, 0.f, 0.f};          // four partial sums: a quarter of the chain of dependent additions
#pragma unroll
      for (int ii = 0; ii < DS; ii += 4) {
        const float4 f4 = pf[ii / 4], q4 = pq[ii / 4];
        S[ii] = f4.x * S[ii] + (1.f - f4.x) * vj;
        S[ii + 1] = f4.y * S[ii + 1] + (1.f - f4.y) * vj;
        S[ii + 2] = f4.z * S[ii + 2] + (1.f - f4.z) * vj;
        S[ii + 3] = f4.w * S[ii + 3] + (1.f - f4.w) * vj;
        nm[0] += S[ii] * q4.x;
        nm[1] += S[ii + 1] * q4.y;
        nm[2] += S[ii + 2] * q4.z;
        nm[3] += S[ii + 3] * q4.w;
      }
      const float num = lanes_sum<SP>((nm[0] + nm[1]) + (nm[2] + nm[3]));
      if (live && part == 0) so[tt * Dv + col] = num;
    }
    __syncthreads();
    for (int tt = wave; tt < n; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < Dv; i += 64) ss += so[tt * Dv + i] * so[tt * Dv + i];
      ss = wave_sum(ss);
      if (lane == 0) sinv[tt] = 1.f / sqrtf(ss / (float)Dv + eps);
    }
    __syncthreads();
    if (live) {
#pragma unroll
      for (int u = 0; u < PERV; ++u) {
        const int tt = part + u * SP;
        if (tt < n) E::store(out, (start + c0 + tt) * out_stride + colv + col, so[tt * Dv + col] * sinv[tt] * nw);
      }
    }
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < DS; ++ii) {
      const int i = part * DS + ii;
      if (i < D) st[(int64_t)i * Dv + col] = S[ii];
    }
  }
}

template <typename Tag>
static int launch_hgrn2(void* out, int64_t out_stride, const void* qpre, int64_t q_stride, const void* fpre, int64_t f_stride,
                        const void* v, int64_t v_stride, const float* f_bias, const float* lower, const float* norm_w,
                        float* state, int64_t state_stride, const SeqBatch& s, int H, int D, int Dv, float eps,
                        hipStream_t st) {
  const dim3 grid((unsigned)s.B, (unsigned)H);
  // (register rows past D take f = 0 and q = 0: whatever they hold never reaches an output and is never stored)
  // workgroup sizes come in steps (the staging's trip count is a compile-time number): the next one that holds Dv columns
#define SP_HGRN_NT(DP, SP, NT)                                                                                          \
  hgrn2_scan_kernel<Tag, DP, SP, NT><<<grid, NT, (size_t)hgrn_chunk(DP) * 2 * Dv * sizeof(float), st>>>(                \
      out, out_stride, qpre, q_stride, fpre, f_stride, v, v_stride, f_bias, lower, norm_w, state, state_stride, s, H, D, Dv, eps)
#define SP_HGRN_SP(DP, SP)                                                                                              \
  do {                                                                                                                  \
    const int need = Dv * SP;                                                                                           \
    if (need <= 64) SP_HGRN_NT(DP, SP, 64);                                                                             \
    else if (need <= 128) SP_HGRN_NT(DP, SP, 128);                                                                      \
    else if (need <= 256) SP_HGRN_NT(DP, SP, 256);                                                                      \
    else if (need <= 512) SP_HGRN_NT(DP, SP, 512);                                                                      \
    else SP_HGRN_NT(DP, SP, 1024);                                                                                      \
  } while (0)
#define SP_HGRN(DP)                                                                                                     \
  do {                                                                                                                  \
    if (Dv * hgrn_split_fine(DP) <= 1024) SP_HGRN_SP(DP, hgrn_split_fine(DP));                                          \
    else if (Dv * hgrn_split_coarse(DP) <= 1024) SP_HGRN_SP(DP, hgrn_split_coarse(DP));                                 \
    else return SP_ERR_UNSUPPORTED;                                                                                     \
  } while (0)
  if (D <= 16) SP_HGRN(16);
  else if (D <= 32) SP_HGRN(32);
  else if (D <= 64) SP_HGRN(64);
  else if (D <= 128) SP_HGRN(128);
  else if (D <= 256) SP_HGRN(256);
  else return SP_ERR_UNSUPPORTED;
#undef SP_HGRN
#undef SP_HGRN_SP
#undef SP_HGRN_NT
  SP_LAUNCH_CHECK();
  return SP_OK;
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_hgrn2_scan(void* out, int64_t out_stride, const void* qpre, int64_t q_stride, const void* fpre,
                             int64_t f_stride, const void* v, int64_t v_stride, const float* f_bias, const float* lower,
                             const float* norm_w, float* state, int64_t state_stride, int heads, int dim, int vdim, float eps,
                             SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && heads > 0 && dim > 0 && vdim > 0 && vdim <= 256);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(out && qpre && fpre && v && f_bias && lower && norm_w && state && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  const int64_t nk = (int64_t)heads * dim, nv = (int64_t)heads * vdim;
  SP_CHECK_ARG(q_stride >= nk && f_stride >= nk && v_stride >= nv && out_stride >= nv && state_stride >= nk * vdim);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, return (launch_hgrn2<Tag>(out, out_stride, qpre, q_stride, fpre, f_stride, v, v_stride, f_bias, lower,
                                                     norm_w, state, state_stride, s, heads, dim, vdim, eps,
                                                     (hipStream_t)stream)));
}
