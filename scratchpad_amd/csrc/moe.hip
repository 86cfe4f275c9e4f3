// Mixture of experts: fp32 router with sigmoid scores, a choice correction and group-limited top-k; the (token, expert)
// pairs of a step ordered by expert on the device; a grouped matrix product over that order (every expert's weights are
// read once per row tile, fp32 accumulation); the clamped gated activation; and the weighted sum of a token's experts in
// a fixed order, so a token's result does not depend on which other tokens share the step.
#include "seq_batch.h"

namespace sp {
namespace {

// ---- router: one wave per token ----------------------------------------------------------------------------------
// z = W x (fp32), s = sigmoid(z), choice = s + correction; groups: score = sum of the two largest choices of the group,
// the best `keep` groups stay, the others' choices count as -inf; the `top` largest choices win; weights = their s.
template <typename Tag>
__global__ void moe_route_kernel(int32_t* ids, float* weights, const void* x, int64_t x_stride, const float* router,
                                 const float* correction, int64_t T, int width, int E, int top, int groups, int keep) {
  typedef Elem<Tag> El;
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
  if (t >= T) return;
  float* score = smem + (size_t)wave * (2 * E + groups);     // s[E], choice[E], group score[groups]
  float* choice = score + E;
  float* gscore = choice + E;
  for (int e = 0; e < E; ++e) {
    float d = 0.f;
    for (int i = lane; i < width; i += 64) d += router[(int64_t)e * width + i] * El::load(x, t * x_stride + i);
    d = wave_sum(d);
    if (lane == 0) {
      const float sg = 1.f / (1.f + expf(-d));
      score[e] = sg;
      choice[e] = sg + correction[e];
    }
  }
  __builtin_amdgcn_wave_barrier();
  if (groups > 1 && keep < groups) {
    const int per = E / groups;
    for (int gidx = lane; gidx < groups; gidx += 64) {
      float a = -INFINITY, b2 = -INFINITY;              // the two largest
      for (int e = gidx * per; e < (gidx + 1) * per; ++e) {
        const float c = choice[e];
        if (c > a) { b2 = a; a = c; }
        else if (c > b2) b2 = c;
      }
      gscore[gidx] = per > 1 ? a + b2 : a;
    }
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) {
      // drop all but the best `keep` groups (ties: the lower index stays)
      for (int gidx = 0; gidx < groups; ++gidx) {
        int better = 0;
        for (int o = 0; o < groups; ++o)
          better += (gscore[o] > gscore[gidx]) || (gscore[o] == gscore[gidx] && o < gidx);
        if (better >= keep)
          for (int e = gidx * per; e < (gidx + 1) * per; ++e) choice[e] = -INFINITY;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c > best || (c == best && e < at && c > -INFINITY)) { best = c; at = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = 0;                                  // fewer finite choices than `top`: cannot happen for top <= kept experts
    if (lane == 0) {
      ids[t * top + k] = at;
      weights[t * top + k] = score[at];
      choice[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- softmax scores and choice on ready fp32 logits: one wave per token ---------------------------------------------
// s = softmax(z) over all experts; the `top` largest s win (ties: the lower index); weights = s * scale
__global__ void moe_softmax_topk_kernel(int32_t* ids, float* weights, const float* logits, int64_t T, int E, int top,
                                        float scale, int renorm) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
  if (t >= T) return;
  float* score = smem + (size_t)wave * 2 * E;     // s[E], then the choice copy
  float* choice = score + E;
  float zmax = -INFINITY;
  for (int e = lane; e < E; e += 64) zmax = fmaxf(zmax, logits[t * E + e]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) zmax = fmaxf(zmax, __shfl_xor(zmax, off, 64));
  float part = 0.f;
  for (int e = lane; e < E; e += 64) part += expf(logits[t * E + e] - zmax);
  const float inv = 1.f / wave_sum(part);
  for (int e = lane; e < E; e += 64) {
    const float sv = expf(logits[t * E + e] - zmax) * inv;
    score[e] = sv;
    choice[e] = sv;
  }
  __builtin_amdgcn_wave_barrier();
  float chosen = 0.f;                                  // lane 0: the sum of the chosen scores
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c > best) { best = c; at = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = 0;
    if (lane == 0) {
      ids[t * top + k] = at;
      weights[t * top + k] = score[at] * scale;
      chosen += score[at];
      choice[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  // the softmax over the chosen logits only = the chosen scores divided by their sum
  if (renorm && lane == 0)
    for (int k = 0; k < top; ++k) weights[t * top + k] /= chosen;
}

// ---- pairs ordered by expert: offsets[E + 1], order[pos] = pair, place[pair] = pos.  One workgroup. ---------------
__global__ void moe_align_kernel(int32_t* offsets, int32_t* order, int32_t* place, const int32_t* ids, int P, int E) {
  extern __shared__ int32_t cnt[];          // counts[E], then cursors[E]
  int32_t* cur = cnt + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&cnt[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = run;
      cur[e] = run;
      run += cnt[e];
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int pos = atomicAdd(&cur[ids[p]], 1);
    order[pos] = p;
    place[p] = pos;
  }
}

// ---- grouped product: out[pos, n] = sum_k a[row(pos), k] * w[expert(pos), n, k] -------------------------------------
// row(pos) = order[pos] / row_div when order is given (the token of a pair), else pos.  Tiles of 32 rows x 64 columns;
// a tile never spans two experts.  Each output element accumulates over k in the same order wherever its row sits.
constexpr int GM = 32, GN = 64, GK = 32;

template <typename Tag>
__global__ void __launch_bounds__(256)
moe_grouped_gemm_kernel(void* out, const void* a, const void* w, const int32_t* offsets, const int32_t* order, int row_div,
                        int P, int N, int K, int E, int64_t a_stride, int64_t out_stride) {
  typedef Elem<Tag> El;
  __shared__ float As[GK][GM + 1];
  __shared__ float Bs[GK][GN + 4];
  // which expert and which of its row tiles
  int tile = blockIdx.x, e = 0, row0 = 0, rows_end = 0;
  for (; e < E; ++e) {
    const int lo = offsets[e], hi = offsets[e + 1];
    const int tiles = (hi - lo + GM - 1) / GM;
    if (tile < tiles) {
      row0 = lo + tile * GM;
      rows_end = hi;
      break;
    }
    tile -= tiles;
  }
  if (e >= E) return;
  const int n0 = blockIdx.y * GN;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;       // 16 x 16 threads: 2 rows x 4 columns each
  float acc[2][4] = {};
  const char* wbase = (const char*)w + (int64_t)e * N * K * El::kBytes;
  // loader roles: A tile 32 x 32 (4 per thread), B tile 64 x 32 (8 per thread)
  const int ar = threadIdx.x >> 3, ak = (threadIdx.x & 7) * 4;
  const int br = threadIdx.x >> 2, bk = (threadIdx.x & 3) * 8;
  int64_t arow = -1;
  if (row0 + ar < rows_end) arow = order ? order[row0 + ar] / row_div : row0 + ar;
  for (int k0 = 0; k0 < K; k0 += GK) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + ak + i;
      As[ak + i][ar] = (arow >= 0 && k < K) ? El::load(a, arow * a_stride + k) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + bk + i, n = n0 + br;
      Bs[bk + i][br] = (n < N && k < K) ? El::load(wbase, (int64_t)n * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      const float a0 = As[k][ty * 2], a1 = As[k][ty * 2 + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float bv = Bs[k][tx * 4 + j];
        acc[0][j] += a0 * bv;
        acc[1][j] += a1 * bv;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int pos = row0 + ty * 2 + i;
    if (pos >= rows_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) El::store(out, (int64_t)pos * out_stride + n, acc[i][j]);
    }
  }
}

// ---- the same product on the matrix cores (16-bit types, K a multiple of 32, 16-byte aligned rows) -------------------
// Tiles of 128 rows x 64 columns, 4 waves of 32 x 64 each: per k-step of 32 a wave loads 2 row fragments and 4 weight
// fragments (16 bytes per lane, straight from global memory: the 4 waves of a workgroup share the weight fragments
// through the cache) and issues 8 MFMAs.  v_mfma_f32_16x16x32: lane (r16 = lane & 15, q = lane >> 4) holds 8 k-values of
// row r16 of each operand and receives D[4 q + r][r16], r < 4 - with the weights as the first operand a lane ends up
// with 4 neighbouring output columns of ONE row.  A wave whose 32 rows lie past the expert's rows leaves at once, so a
// decode step (a few rows per expert) streams every chosen expert's weights once and does little else.
typedef float f32x4_q __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_q __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_q __attribute__((ext_vector_type(8)));
template <typename Tag>
__device__ __forceinline__ f32x4_q mfma_q(const u32x4& a, const u32x4& b, const f32x4_q& c);
template <>
__device__ __forceinline__ f32x4_q mfma_q<bf16_tag>(const u32x4& a, const u32x4& b, const f32x4_q& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_q, a), __builtin_bit_cast(bf16x8_q, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_q mfma_q<f16_tag>(const u32x4& a, const u32x4& b, const f32x4_q& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_q, a), __builtin_bit_cast(f16x8_q, b), c, 0, 0, 0);
}

constexpr int QM = 128, QN = 64;

template <typename Tag>
__global__ void __launch_bounds__(256)
moe_grouped_mfma_kernel(void* out, const void* a, const void* w, const int32_t* offsets, const int32_t* order, int row_div,
                        int N, int K, int E, int64_t a_stride, int64_t out_stride) {
  typedef Elem<Tag> El;
  int tile = blockIdx.x, e = 0, row0 = 0, rows_end = 0;
  for (; e < E; ++e) {
    const int lo = offsets[e], hi = offsets[e + 1];
    const int tiles = (hi - lo + QM - 1) / QM;
    if (tile < tiles) {
      row0 = lo + tile * QM;
      rows_end = hi;
      break;
    }
    tile -= tiles;
  }
  if (e >= E) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, q = lane >> 4;
  if (row0 + 32 * wave >= rows_end) return;                       // (no workgroup barrier in this kernel)
  const int n0 = blockIdx.y * QN;
  const char* xp[2];
  bool xv[2];
#pragma unroll
  for (int f = 0; f < 2; ++f) {
    const int pos = row0 + 32 * wave + 16 * f + r16;
    xv[f] = pos < rows_end;
    const int64_t arow = xv[f] ? (order ? order[pos] / row_div : pos) : 0;
    xp[f] = (const char*)a + (arow * a_stride + 8 * q) * 2;
  }
  const char* wbase = (const char*)w + (int64_t)e * N * K * 2;
  const char* wp[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = min(n0 + 16 * j + r16, N - 1);                  // columns past N are computed and never stored
    wp[j] = wbase + ((int64_t)n * K + 8 * q) * 2;
  }
  f32x4_q acc[2][4];
#pragma unroll
  for (int f = 0; f < 2; ++f)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[f][j] = f32x4_q{0.f, 0.f, 0.f, 0.f};
  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (int k0 = 0; k0 < K; k0 += 32) {
    u32x4 xf[2], wf[4];
#pragma unroll
    for (int f = 0; f < 2; ++f) xf[f] = xv[f] ? ld16(xp[f] + (int64_t)k0 * 2) : zero;
#pragma unroll
    for (int j = 0; j < 4; ++j) wf[j] = ld16(wp[j] + (int64_t)k0 * 2);
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[f][j] = mfma_q<Tag>(wf[j], xf[f], acc[f][j]);
  }
#pragma unroll
  for (int f = 0; f < 2; ++f) {
    const int pos = row0 + 32 * wave + 16 * f + r16;
    if (pos >= rows_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + 16 * j + 4 * q + r;
        if (n < N) El::store(out, (int64_t)pos * out_stride + n, acc[f][j][r]);
      }
  }
}

// ---- y = g' * sigmoid(alpha g') * (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit); gu = [g | u] per row -----
template <typename Tag>
__global__ void moe_glu_kernel(void* out, const void* gu, int64_t P, int F, float limit, float alpha) {
  typedef Elem<Tag> El;
  const int64_t n = P * (int64_t)F;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t p = i / F;
    const int f = (int)(i % F);
    const float g = fminf(El::load(gu, p * 2 * F + f), limit);
    const float u = fminf(fmaxf(El::load(gu, p * 2 * F + F + f), -limit), limit);
    El::store(out, i, g / (1.f + expf(-alpha * g)) * (u + 1.f));
  }
}

// ---- out[t] = sum_k weights[t, k] * z[place[t * top + k]] ----------------------------------------------------------
template <typename Tag>
__global__ void moe_combine_kernel(void* out, const void* z, const int32_t* place, const float* weights, int width,
                                   int top, int64_t out_stride) {
  typedef Elem<Tag> El;
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc += weights[t * top + k] * El::load(z, (int64_t)place[t * top + k] * width + i);
    El::store(out, t * out_stride + i, acc);
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_moe_route(int32_t* ids, float* weights, const void* x, int64_t x_stride, const float* router,
                            const float* correction, int64_t num_tokens, int width, int experts, int top, int groups,
                            int keep, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && experts > 0 && top > 0 && top <= experts);
  SP_CHECK_ARG(groups >= 1 && keep >= 1 && keep <= groups && experts % groups == 0);
  SP_CHECK_ARG((int64_t)top <= (int64_t)keep * (experts / groups));
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(ids && weights && x && router && correction && x_stride >= width);
  const size_t lds = 4 * (size_t)(2 * experts + groups) * sizeof(float);
  if (lds > 64 * 1024) return SP_ERR_UNSUPPORTED;
  SP_DISPATCH_DTYPE(dtype, (moe_route_kernel<Tag><<<dim3((unsigned)((num_tokens + 3) / 4)), 256, lds, (hipStream_t)stream>>>(
                               ids, weights, x, x_stride, router, correction, num_tokens, width, experts, top, groups, keep)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_moe_softmax_topk(int32_t* ids, float* weights, const float* logits, int64_t num_tokens, int experts, int top,
                                   float scale, int renorm, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && experts > 0 && top > 0 && top <= experts);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(ids && weights && logits);
  const size_t lds = 4 * (size_t)(2 * experts) * sizeof(float);
  if (lds > 64 * 1024) return SP_ERR_UNSUPPORTED;
  moe_softmax_topk_kernel<<<dim3((unsigned)((num_tokens + 3) / 4)), 256, lds, (hipStream_t)stream>>>(ids, weights, logits,
                                                                                                  num_tokens, experts, top, scale,
                                                                                                  renorm);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_moe_align(int32_t* offsets, int32_t* order, int32_t* place, const int32_t* ids, int pairs, int experts,
                            void* stream) {
  SP_CHECK_ARG(pairs >= 0 && experts > 0 && experts <= 4096);
  SP_CHECK_ARG(offsets && (pairs == 0 || (order && place && ids)));
  moe_align_kernel<<<1, 1024, 2 * (size_t)experts * sizeof(int32_t), (hipStream_t)stream>>>(offsets, order, place, ids,
                                                                                            pairs, experts);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_moe_grouped_gemm(void* out, const void* a, const void* w, const int32_t* offsets, const int32_t* order,
                                   int row_div, int pairs, int n, int k, int experts, int64_t a_stride,
                                   int64_t out_stride, int dtype, void* stream) {
  SP_CHECK_ARG(pairs >= 0 && n > 0 && k > 0 && experts > 0 && row_div >= 1);
  if (pairs == 0) return SP_OK;
  SP_CHECK_ARG(out && a && w && offsets && a_stride >= k && out_stride >= n);
  const bool aligned = k % 32 == 0 && a_stride % 8 == 0 && ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0;
  if ((dtype == SP_BF16 || dtype == SP_F16) && aligned) {
    const dim3 grid((unsigned)((pairs + QM - 1) / QM + experts), (unsigned)((n + QN - 1) / QN));
    if (dtype == SP_BF16)
      moe_grouped_mfma_kernel<bf16_tag><<<grid, 256, 0, (hipStream_t)stream>>>(out, a, w, offsets, order, row_div, n, k,
                                                                                experts, a_stride, out_stride);
    else
      moe_grouped_mfma_kernel<f16_tag><<<grid, 256, 0, (hipStream_t)stream>>>(out, a, w, offsets, order, row_div, n, k,
                                                                               experts, a_stride, out_stride);
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  const dim3 grid((unsigned)((pairs + GM - 1) / GM + experts), (unsigned)((n + GN - 1) / GN));
  SP_DISPATCH_DTYPE(dtype, (moe_grouped_gemm_kernel<Tag><<<grid, 256, 0, (hipStream_t)stream>>>(
                               out, a, w, offsets, order, row_div, pairs, n, k, experts, a_stride, out_stride)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_moe_glu(void* out, const void* gu, int64_t pairs, int ff, float limit, float alpha, int dtype,
                          void* stream) {
  SP_CHECK_ARG(pairs >= 0 && ff > 0);
  if (pairs == 0) return SP_OK;
  SP_CHECK_ARG(out && gu);
  int64_t blocks = (pairs * ff + kBlock - 1) / kBlock;
  if (blocks > 4096) blocks = 4096;
  SP_DISPATCH_DTYPE(dtype, (moe_glu_kernel<Tag><<<dim3((unsigned)blocks), kBlock, 0, (hipStream_t)stream>>>(out, gu, pairs, ff,
                                                                                                         limit, alpha)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_moe_combine(void* out, const void* z, const int32_t* place, const float* weights, int64_t num_tokens,
                              int width, int top, int64_t out_stride, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && top > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && z && place && weights && out_stride >= width);
  SP_DISPATCH_DTYPE(dtype, (moe_combine_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               out, z, place, weights, width, top, out_stride)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}
