// Grouped-query attention over a sliding window plus pooled blocks, on a token-level key/value pool.
//
// A query at position p sees the tokens j with 0 <= p - j < size and, for every block of P consecutive positions that
// lies wholly before the window (block b = positions bP .. bP + P - 1, seen once bP + P - 1 <= p - size), ONE key and
// value: the means of the block's cached keys and values.  Tokens and blocks share one softmax.  Tokens that left the
// window while their block is still incomplete behind it are not seen.  size <= 0 means no window (plain causal),
// P <= 0 no pooling.
//
// Cache: per token a key row [G, D] (rotated) and a value row [G, Dv] (each head divided by its root mean square); the
// pooled key/value of block b lives in a second pair of buffers at the slot of the block's LAST token, written by the
// step that brings this token, so the pooled rows need no allocator of their own and are freed with the token.
//
// Rotation: "rotate half" - coordinate i < dims/2 pairs with i + dims/2 - or, with `adjacent`, coordinate 2i with 2i + 1;
// angle = position * freq[i] in fp32, cos and sin times mag; coordinates from dims on pass.  Optional fp32 biases join q, k
// and v before the rotation; the per-head norm of the values can be switched off.  Scores, softmax and the weighted sum are
// fp32.  With `sinks` (one fp32 number per query head) the softmax's denominator holds one more term exp(sink): a key that
// is seen by every query, is not scaled and has no value.
//
// Further forms of the same layer (each a parameter): q and k divided per head by their root mean square after the
// rotation; q times a number per head and times 1 + coef ln(floor((position + 1) / every) + 1); values blended with the
// values an earlier layer cached for the same token, v <- (1 - lambda) v + lambda v_first; scores capped as
// cap tanh(score / cap); and, instead of the softmax, every visible key weighted by sigmoid(score + bias[head]) without
// normalisation.  The result can be multiplied element by element with sigmoid(gate) on its way out.
#include "seq_batch.h"

namespace sp {
namespace {

// q rotated in place; k rotated and v (normed per head unless norm_v is 0) into the pool rows loc[t]
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
qkv_rotary_store_kernel(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                        void* kpool, int64_t kp_stride, void* vpool, int64_t vp_stride, const int64_t* positions,
                        const int64_t* loc, const float* freq, float mag, const float* qb, const float* kb, const float* vb,
                        int H, int G, int D, int Dv, int dims, int adjacent, int norm_v, float eps) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = dims / 2;
  const int64_t slot = loc[t];
  const int second = adjacent ? 1 : half, step = adjacent ? 2 : 1;      // a pair is (i * step, i * step + second)
  for (int e = threadIdx.x; e < H * half; e += blockDim.x) {
    const int h = e / half, i = e % half;
    const float a = pos * freq[i];
    const float c = cosf(a) * mag, sn = sinf(a) * mag;
    const int col = h * D + i * step;
    const int64_t at = t * q_stride + col;
    const float u = E::load(q, at) + (qb ? qb[col] : 0.f), w = E::load(q, at + second) + (qb ? qb[col + second] : 0.f);
    E::store(q, at, u * c - w * sn);
    E::store(q, at + second, w * c + u * sn);
  }
  for (int e = threadIdx.x; e < G * half; e += blockDim.x) {
    const int g = e / half, i = e % half;
    const float a = pos * freq[i];
    const float c = cosf(a) * mag, sn = sinf(a) * mag;
    const int col = g * D + i * step;
    const int64_t at = t * k_stride + col, to = slot * kp_stride + col;
    const float u = E::load(k, at) + (kb ? kb[col] : 0.f), w = E::load(k, at + second) + (kb ? kb[col + second] : 0.f);
    E::store(kpool, to, u * c - w * sn);
    E::store(kpool, to + second, w * c + u * sn);
  }
  const int rest = D - dims;
  if (qb)
    for (int e = threadIdx.x; e < H * rest; e += blockDim.x) {
      const int col = (e / rest) * D + dims + e % rest;
      E::store(q, t * q_stride + col, E::load(q, t * q_stride + col) + qb[col]);
    }
  for (int e = threadIdx.x; e < G * rest; e += blockDim.x) {
    const int col = (e / rest) * D + dims + e % rest;
    E::store(kpool, slot * kp_stride + col, E::load(k, t * k_stride + col) + (kb ? kb[col] : 0.f));
  }
  if (!norm_v) {
    for (int e = threadIdx.x; e < G * Dv; e += blockDim.x)
      E::store(vpool, slot * vp_stride + e, E::load(v, t * v_stride + e) + (vb ? vb[e] : 0.f));
    return;
  }
  // value heads: one wave each
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int g = wave; g < G; g += waves) {
    const int64_t at = t * v_stride + (int64_t)g * Dv, to = slot * vp_stride + (int64_t)g * Dv;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += 64) {
      const float x = E::load(v, at + i) + (vb ? vb[g * Dv + i] : 0.f);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
    for (int i = lane; i < Dv; i += 64) E::store(vpool, to + i, (E::load(v, at + i) + (vb ? vb[g * Dv + i] : 0.f)) * inv);
  }
}

// The same store with a wave per head: q and k can be divided by their root mean square over the head AFTER the rotation
// (qk_norm), q scaled per head and by position, v blended with the row another layer's pool holds for the same slot.
// A lane holds the coordinates lane, lane + 64, ... of its head (dim, vdim <= 64 * kStorePerLane).
constexpr int kStorePerLane = 4;
template <typename Tag>
__device__ __forceinline__ void rotated_head(float* val, const void* src, int64_t at, const float* bias, int col0, int D,
                                             int dims, int adjacent, float pos, const float* freq, float mag, int lane) {
  typedef Elem<Tag> E;
  const int half = dims / 2;
#pragma unroll
  for (int u = 0; u < kStorePerLane; ++u) {
    const int i = lane + 64 * u;
    float out = 0.f;
    if (i < D) {
      const float x = E::load(src, at + i) + (bias ? bias[col0 + i] : 0.f);
      out = x;
      if (i < dims) {
        int pi, fi;
        bool first;
        if (adjacent) {
          first = (i & 1) == 0;
          pi = first ? i + 1 : i - 1;
          fi = i >> 1;
        } else {
          first = i < half;
          pi = first ? i + half : i - half;
          fi = first ? i : i - half;
        }
        const float y = E::load(src, at + pi) + (bias ? bias[col0 + pi] : 0.f);
        const float ang = pos * freq[fi];
        const float c = cosf(ang) * mag, sn = sinf(ang) * mag;
        out = first ? x * c - y * sn : x * c + y * sn;
      }
    }
    val[u] = out;
  }
}

template <typename Tag>
__global__ void __launch_bounds__(kBlock)
qkv_norm_store_kernel(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                      void* kpool, int64_t kp_stride, void* vpool, int64_t vp_stride, const int64_t* positions,
                      const int64_t* loc, const float* freq, float mag, const float* qb, const float* kb, const float* vb,
                      int H, int G, int D, int Dv, int dims, int adjacent, int norm_v, float eps, int qk_norm,
                      const float* q_head_scale, float q_temp_coef, int q_temp_every, const void* v_first,
                      int64_t vf_stride, const float* v_mix) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  const int64_t ipos = positions[t];
  const float pos = (float)ipos;
  const int64_t slot = loc[t];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  float qmul = 1.f;
  if (q_temp_every > 0) qmul = 1.f + q_temp_coef * logf((float)((ipos + 1) / q_temp_every) + 1.f);
  for (int job = wave; job < H + 2 * G; job += waves) {
    float val[kStorePerLane];
    if (job < H + G) {
      const bool isq = job < H;
      const int h = isq ? job : job - H;
      const void* src = isq ? q : k;
      const int64_t at = t * (isq ? q_stride : k_stride) + (int64_t)h * D;
      rotated_head<Tag>(val, src, at, isq ? qb : kb, h * D, D, dims, adjacent, pos, freq, mag, lane);
      float mul = 1.f;
      if (qk_norm) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < kStorePerLane; ++u) ss += val[u] * val[u];       // (coordinates past D are zeros)
        ss = wave_sum(ss);
        mul = 1.f / sqrtf(ss / (float)D + eps);
      }
      if (isq) mul *= qmul * (q_head_scale ? q_head_scale[h] : 1.f);
      void* dst = isq ? q : kpool;
      const int64_t to = isq ? at : slot * kp_stride + (int64_t)h * D;
#pragma unroll
      for (int u = 0; u < kStorePerLane; ++u) {
        const int i = lane + 64 * u;
        if (i < D) E::store(dst, to + i, val[u] * mul);
      }
    } else {
      const int g = job - H - G;
      const int64_t at = t * v_stride + (int64_t)g * Dv, to = slot * vp_stride + (int64_t)g * Dv;
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < kStorePerLane; ++u) {
        const int i = lane + 64 * u;
        val[u] = i < Dv ? E::load(v, at + i) + (vb ? vb[g * Dv + i] : 0.f) : 0.f;
        ss += val[u] * val[u];
      }
      float mul = 1.f;
      if (norm_v) mul = 1.f / sqrtf(wave_sum(ss) / (float)Dv + eps);
      const float lam = v_first ? v_mix[0] : 0.f;
#pragma unroll
      for (int u = 0; u < kStorePerLane; ++u) {
        const int i = lane + 64 * u;
        if (i < Dv) {
          float x = val[u] * mul;
          if (v_first) x = (1.f - lam) * x + lam * E::load(v_first, slot * vf_stride + (int64_t)g * Dv + i);
          E::store(vpool, to + i, x);
        }
      }
    }
  }
}

// a token that completes a block (position + 1 divisible by P) writes the block's mean key and value at its own slot
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
pool_blocks_kernel(void* kpooled, void* vpooled, const void* kpool, const void* vpool, int64_t kp_stride, int64_t vp_stride,
                   const int32_t* req_to_token, int64_t table_stride, SeqBatch s, int kw, int vw, int P) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const int64_t pos = prefix + (t - start);
  if ((pos + 1) % P != 0) return;
  const int32_t* table = req_to_token + load_idx(s.req_pool_indices, b, s.idx64) * table_stride;
  const int64_t first = pos - P + 1, dst = table[pos];
  const float inv = 1.f / (float)P;
  for (int c = threadIdx.x; c < kw + vw; c += blockDim.x) {
    const bool isk = c < kw;
    const void* src = isk ? kpool : vpool;
    const int64_t stride = isk ? kp_stride : vp_stride;
    const int col = isk ? c : c - kw;
    float acc = 0.f;
    for (int j = 0; j < P; ++j) acc += E::load(src, (int64_t)table[first + j] * stride + col);
    E::store(isk ? kpooled : vpooled, dst * stride + col, acc * inv);
  }
}

constexpr int kMaxPerLane = 4;       // value width Dv <= 64 * kMaxPerLane

template <typename Tag, bool VEC>
__device__ __forceinline__ float dot_row(const float* sq, const void* base, int64_t at, int D) {
  typedef Elem<Tag> E;
  float d = 0.f;
  if (VEC) {
    constexpr int V = E::kVec;
    for (int i = 0; i < D; i += V) {
      float f[V];
      unpack16<Tag>(ld16((const char*)base + (at + i) * E::kBytes), f);
#pragma unroll
      for (int e = 0; e < V; ++e) d += sq[i + e] * f[e];
    }
  } else {
    for (int i = 0; i < D; ++i) d += sq[i] * E::load(base, at + i);
  }
  return d;
}

// One workgroup of NW waves per (token, query head) - 4 for the rows of prompts, 16 for single decoded tokens, where the
// rows are few and each is long.  The query's keys are numbered blocks first, then the window's tokens, in tiles of 64;
// wave w takes tiles w, w + NW, ...: lane = key for the scores, lane = value channel for the
// weighted sum (4 keys' rows in flight at a time); the waves' partial (maximum, sum, weighted values) meet in LDS.
// The order of every sum depends on the query's position only, never on the batch or on how the prompt was cut.
template <typename Tag, bool VEC, bool SIG>
__global__ void __launch_bounds__(1024)
window_attention_kernel(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kpool, const void* vpool,
                        const void* kpooled, const void* vpooled, int64_t kp_stride, int64_t vp_stride,
                        const int32_t* req_to_token, int64_t table_stride, SeqBatch s, int H, int G, int D, int Dv,
                        int64_t size, int P, float scale, const float* sinks, float softcap, const float* head_bias,
                        const void* gate, int64_t gate_stride) {
  typedef Elem<Tag> E;
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, NW = blockDim.x >> 6;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  float* sq = smem;                              // [D] the scaled query
  float* sw = smem + D + wave * 64;              // this wave's 64 weights
  float* sacc = smem + D + 64 * NW;              // [NW][Dv]
  float* sml = sacc + NW * Dv;                   // [NW] maxima, [NW] sums
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const int64_t pos = prefix + (t - start);
  const int64_t w0 = (size > 0 && pos - size + 1 > 0) ? pos - size + 1 : 0;      // first token of the window
  const int64_t nb = (size > 0 && P > 0) ? w0 / P : 0;                            // blocks wholly before it
  const int64_t total = nb + (pos - w0 + 1);
  const int g = h / (H / G);
  const int32_t* table = req_to_token + load_idx(s.req_pool_indices, b, s.idx64) * table_stride;
  for (int i = threadIdx.x; i < D; i += blockDim.x) sq[i] = E::load(q, t * q_stride + (int64_t)h * D + i) * scale;
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  const float hbias = (SIG && head_bias) ? head_bias[h] : 0.f;
  float acc[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) acc[i] = 0.f;
  const int64_t vcol = (int64_t)g * Dv;
  for (int64_t k0 = (int64_t)wave * 64; k0 < total; k0 += 64 * NW) {
    const int n = (int)(total - k0 < 64 ? total - k0 : 64);
    float sc = -INFINITY;
    if (lane < n) {
      const int64_t kk = k0 + lane;
      const bool blk = kk < nb;
      const int64_t row = blk ? table[kk * P + P - 1] : table[w0 + (kk - nb)];
      sc = dot_row<Tag, VEC>(sq, blk ? kpooled : kpool, row * kp_stride + (int64_t)g * D, D);
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
    }
    if constexpr (SIG) {                                // every visible key on its own: no maximum, no denominator
      sw[lane] = lane < n ? 1.f / (1.f + expf(-(sc + hbias))) : 0.f;
      __builtin_amdgcn_wave_barrier();
    } else {
      float tm = sc;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) tm = fmaxf(tm, __shfl_xor(tm, off, 64));
      const float m_new = fmaxf(m, tm);
      const float corr = expf(m - m_new);                 // first tile: exp(-inf) = 0
      const float p = lane < n ? expf(sc - m_new) : 0.f;
      l = l * corr + wave_sum(p);
      m = m_new;
      sw[lane] = p;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) acc[i] *= corr;
    }
    int j = 0;
    for (; j + 4 <= n; j += 4) {
      int64_t at[4];
      const void* src[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t kk = k0 + j + u;
        const bool blk = kk < nb;
        at[u] = (int64_t)(blk ? table[kk * P + P - 1] : table[w0 + (kk - nb)]) * vp_stride + vcol;
        src[u] = blk ? vpooled : vpool;
      }
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int c = lane + 64 * i;
        if (c < Dv) {
          const float v0 = E::load(src[0], at[0] + c), v1 = E::load(src[1], at[1] + c);
          const float v2 = E::load(src[2], at[2] + c), v3 = E::load(src[3], at[3] + c);
          acc[i] += sw[j] * v0;
          acc[i] += sw[j + 1] * v1;
          acc[i] += sw[j + 2] * v2;
          acc[i] += sw[j + 3] * v3;
        }
      }
    }
    for (; j < n; ++j) {
      const int64_t kk = k0 + j;
      const bool blk = kk < nb;
      const int64_t at = (int64_t)(blk ? table[kk * P + P - 1] : table[w0 + (kk - nb)]) * vp_stride + vcol;
      const void* src = blk ? vpooled : vpool;
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int c = lane + 64 * i;
        if (c < Dv) acc[i] += sw[j] * E::load(src, at + c);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int c = lane + 64 * i;
    if (c < Dv) sacc[wave * Dv + c] = acc[i];
  }
  if (lane == 0) {
    sml[wave] = m;
    sml[NW + wave] = l;
  }
  __syncthreads();
  if constexpr (SIG) {
    for (int c = threadIdx.x; c < Dv; c += blockDim.x) {
      float num = 0.f;
      for (int w = 0; w < NW; ++w) num += sacc[w * Dv + c];
      if (gate) num /= 1.f + expf(-E::load(gate, t * gate_stride + (int64_t)h * Dv + c));
      E::store(out, t * out_stride + (int64_t)h * Dv + c, num);
    }
    return;
  }
  float M = sml[0];                                                         // wave 0 always holds a key: M is finite
  for (int w = 1; w < NW; ++w) M = fmaxf(M, sml[w]);
  float den = 0.f;
  if (sinks) {                                                              // one more term of the denominator
    M = fmaxf(M, sinks[h]);
    den = expf(sinks[h] - M);
  }
  for (int w = 0; w < NW; ++w) den += sml[NW + w] * expf(sml[w] - M);       // a wave without keys: exp(-inf) = 0
  const float inv = 1.f / den;
  for (int c = threadIdx.x; c < Dv; c += blockDim.x) {
    float num = 0.f;
    for (int w = 0; w < NW; ++w) num += sacc[w * Dv + c] * expf(sml[w] - M);
    num *= inv;
    if (gate) num /= 1.f + expf(-E::load(gate, t * gate_stride + (int64_t)h * Dv + c));
    E::store(out, t * out_stride + (int64_t)h * Dv + c, num);
  }
}


// ---- the same attention on the matrix cores, for portions of prompts in 16-bit types ------------------------------------
// One workgroup per (16 consecutive tokens of one request's portion, key/value head); wave w works for the group's query
// head w (w + 4, ... in further passes).  Keys of the 16 queries' UNION (blocks up to the last query's, tokens from the
// first query's window start to the last query) go by in tiles of 64; who sees what is a mask per (key, query).
//   S^T = K Q^T   v_mfma_f32_16x16x32: first operand = 16 key rows straight from the pool (16 bytes per lane), second =
//                 the query fragment held in registers; a lane receives S^T[key 4q + r][query r16]: four keys of ONE query,
//                 so the softmax of a query is a reduction over r, the tile's four key groups and the lanes q = 0..3.
//   O^T = V^T P^T first operand = V^T from an LDS tile written transposed ([value channel][key], keys contiguous), second =
//                 P^T - exactly the registers the lane already holds: the key order inside a step of 32 is (4q .. 4q + 3 of
//                 the first 16 keys, then of the second 16) for both operands, so P needs no exchange between lanes.
// Scores, softmax and O are fp32; P enters the second product as a 16-bit value plus its 16-bit remainder (two products).
typedef float f32x4_w __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_w __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_w __attribute__((ext_vector_type(8)));
template <typename Tag>
__device__ __forceinline__ f32x4_w mfma_w(const u32x4& a, const u32x4& b, const f32x4_w& c);
template <>
__device__ __forceinline__ f32x4_w mfma_w<bf16_tag>(const u32x4& a, const u32x4& b, const f32x4_w& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_w, a), __builtin_bit_cast(bf16x8_w, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_w mfma_w<f16_tag>(const u32x4& a, const u32x4& b, const f32x4_w& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_w, a), __builtin_bit_cast(f16x8_w, b), c, 0, 0, 0);
}

constexpr int kVtRow = 72;      // 64 keys + 8 of padding per value channel (16-bit elements)

template <typename Tag, int DS, int DT, bool SIG>      // DS = dim / 32, DT = vdim / 16
__global__ void __launch_bounds__(256)
window_attention_mfma_kernel(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kpool,
                             const void* vpool, const void* kpooled, const void* vpooled, int64_t kp_stride, int64_t vp_stride,
                             const int32_t* req_to_token, int64_t table_stride, SeqBatch s, int H, int G, int64_t size, int P,
                             float scale, const float* sinks, float softcap, const float* head_bias, const void* gate,
                             int64_t gate_stride) {
  constexpr int D = 32 * DS, Dv = 16 * DT;
  __shared__ uint16_t vt[Dv][kVtRow];
  __shared__ int32_t sslot[64];
  // which request and which of its 16-row tiles
  int tile = blockIdx.x, b = 0;
  for (; b < s.B; ++b) {
    const int tiles = (s.extend_seq_lens[b] + 15) / 16;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (b >= s.B) return;
  const int g = blockIdx.y, R = H / G;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, qd = lane >> 4;
  const int64_t start = s.extend_start_loc[b], len = s.extend_seq_lens[b], prefix = s.extend_prefix_lens[b];
  const int rows = (int)(len - 16 * tile < 16 ? len - 16 * tile : 16);
  const int64_t t0 = start + 16 * tile, pos0 = prefix + 16 * tile, pos_last = pos0 + rows - 1;
  const int32_t* table = req_to_token + load_idx(s.req_pool_indices, b, s.idx64) * table_stride;
  const bool pooled = size > 0 && P > 0;
  const int64_t w0U = (size > 0 && pos0 - size + 1 > 0) ? pos0 - size + 1 : 0;
  const int64_t w0L = (size > 0 && pos_last - size + 1 > 0) ? pos_last - size + 1 : 0;
  const int64_t nbU = pooled ? w0L / P : 0;
  const int64_t totalU = nbU + (pos_last - w0U + 1);
  // this lane's query (column r16 of every S^T tile)
  const bool qvalid = r16 < rows;
  const int64_t pos_q = pos0 + r16;
  const int64_t w0_q = (size > 0 && pos_q - size + 1 > 0) ? pos_q - size + 1 : 0;
  const int64_t nb_q = pooled ? w0_q / P : 0;
  for (int h0 = 0; h0 < R; h0 += 4) {
    const int hq = g * R + h0 + wave;
    const bool work = h0 + wave < R;
    const float hbias = (SIG && head_bias && work) ? head_bias[hq] : 0.f;
    u32x4 qf[DS];
#pragma unroll
    for (int st = 0; st < DS; ++st)
      qf[st] = (work && qvalid) ? ld16((const char*)q + ((t0 + r16) * q_stride + (int64_t)hq * D + 32 * st + 8 * qd) * 2)
                                : u32x4{0u, 0u, 0u, 0u};
    f32x4_w oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = f32x4_w{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    for (int64_t k0 = 0; k0 < totalU; k0 += 64) {
      __syncthreads();                                   // the previous tile's readers are done
      if (threadIdx.x < 64) {
        const int64_t kk = k0 + threadIdx.x;
        int32_t sl = 0;
        if (kk < totalU) sl = kk < nbU ? table[kk * P + P - 1] : table[w0U + (kk - nbU)];
        sslot[threadIdx.x] = sl;
      }
      __syncthreads();
      // V^T tile: thread = (key, 8 value channels); neighbouring lanes take neighbouring keys (conflict-free 2-byte writes)
      for (int c = threadIdx.x; c < 64 * (Dv / 8); c += 256) {
        const int key = c & 63, dvc = c >> 6;
        const int64_t kk = k0 + key;
        u32x4 val = {0u, 0u, 0u, 0u};
        if (kk < totalU)
          val = ld16((const char*)(kk < nbU ? vpooled : vpool) + ((int64_t)sslot[key] * vp_stride + (int64_t)g * Dv + 8 * dvc) * 2);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w2 = e == 0 ? val[0] : (e == 1 ? val[1] : (e == 2 ? val[2] : val[3]));
          vt[8 * dvc + 2 * e][key] = (uint16_t)(w2 & 0xffffu);
          vt[8 * dvc + 2 * e + 1][key] = (uint16_t)(w2 >> 16);
        }
      }
      __syncthreads();
      if (work) {
        f32x4_w sacc[4];
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
          sacc[sb] = f32x4_w{0.f, 0.f, 0.f, 0.f};
          const int64_t kk = k0 + 16 * sb + r16;         // the key row this lane feeds
          const bool kvalid = kk < totalU;
          const char* kp = (const char*)(kk < nbU ? kpooled : kpool) + ((int64_t)sslot[16 * sb + r16] * kp_stride + (int64_t)g * D + 8 * qd) * 2;
#pragma unroll
          for (int st = 0; st < DS; ++st) {
            const u32x4 a = kvalid ? ld16(kp + 64 * st) : u32x4{0u, 0u, 0u, 0u};
            sacc[sb] = mfma_w<Tag>(a, qf[st], sacc[sb]);
          }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int sb = 0; sb < 4; ++sb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int64_t kk = k0 + 16 * sb + 4 * qd + r;
            bool vis = qvalid && kk < totalU;
            if (vis) {
              if (kk < nbU) vis = kk < nb_q;
              else {
                const int64_t j = w0U + (kk - nbU);
                vis = j >= w0_q && j <= pos_q;
              }
            }
            float v = vis ? sacc[sb][r] * scale : -INFINITY;
            if (vis && softcap > 0.f) v = softcap * tanhf(v / softcap);
            sacc[sb][r] = v;
            mx = fmaxf(mx, v);
          }
        float corr = 1.f;
        float pf[2][8];
        if constexpr (SIG) {                              // sigmoid(score + bias) per visible key, nothing to rescale
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              pf[sb >> 1][4 * (sb & 1) + r] = sacc[sb][r] == -INFINITY ? 0.f : 1.f / (1.f + expf(-(sacc[sb][r] + hbias)));
        } else {
          mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
          mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
          const float m_new = fmaxf(m, mx);
          const float m_safe = m_new == -INFINITY ? 0.f : m_new;      // nothing seen yet: every weight is exp(-inf) = 0
          corr = expf(m - m_safe);
          float psum = 0.f;
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float p = expf(sacc[sb][r] - m_safe);
              psum += p;
              pf[sb >> 1][4 * (sb & 1) + r] = p;
            }
          psum += __shfl_xor(psum, 16, 64);
          psum += __shfl_xor(psum, 32, 64);
          l = l * corr + psum;
          m = m_new;
        }
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          // the weights enter the product as a 16-bit value plus a 16-bit remainder: they are never rounded to 8 bits of
          // mantissa (the second product costs an eighth of the step's matrix work again)
          const u32x4 pb = pack16<Tag>(pf[hh]);
          float rest[8], back[8];
          unpack16<Tag>(pb, back);
#pragma unroll
          for (int e = 0; e < 8; ++e) rest[e] = pf[hh][e] - back[e];
          const u32x4 pr = pack16<Tag>(rest);
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            if (!SIG && hh == 0) {
#pragma unroll
              for (int r = 0; r < 4; ++r) oacc[dt][r] *= corr;
            }
            const u32x2 lo = *(const u32x2*)&vt[16 * dt + r16][32 * hh + 4 * qd];
            const u32x2 hi = *(const u32x2*)&vt[16 * dt + r16][32 * hh + 16 + 4 * qd];
            const u32x4 a = {lo[0], lo[1], hi[0], hi[1]};
            oacc[dt] = mfma_w<Tag>(a, pb, oacc[dt]);
            oacc[dt] = mfma_w<Tag>(a, pr, oacc[dt]);
          }
        }
      }
    }
    if (work && qvalid) {
      float inv = 1.f;
      if constexpr (!SIG) {
        inv = 1.f / l;
        if (sinks) {                                   // (a valid query has seen itself: m is finite)
          const float sk = sinks[hq], m2 = fmaxf(m, sk), keep = expf(m - m2);
          inv = keep / (l * keep + expf(sk - m2));
        }
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        float f[8] = {oacc[dt][0] * inv, oacc[dt][1] * inv, oacc[dt][2] * inv, oacc[dt][3] * inv, 0.f, 0.f, 0.f, 0.f};
        if (gate) {
          float gf[8];
          const u32x2 g2 = *(const u32x2*)((const char*)gate + ((t0 + r16) * gate_stride + (int64_t)hq * Dv + 16 * dt + 4 * qd) * 2);
          unpack16<Tag>(u32x4{g2[0], g2[1], 0u, 0u}, gf);
#pragma unroll
          for (int e = 0; e < 4; ++e) f[e] /= 1.f + expf(-gf[e]);
        }
        const u32x4 pk = pack16<Tag>(f);
        *(u32x2*)((char*)out + ((t0 + r16) * out_stride + (int64_t)hq * Dv + 16 * dt + 4 * qd) * 2) = u32x2{pk[0], pk[1]};
      }
    }
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_qkv_rotary_store(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                   int64_t v_stride, void* kpool, int64_t kp_stride, void* vpool, int64_t vp_stride,
                                   const int64_t* positions, const int64_t* loc, const float* freq, float mag,
                                   const float* q_bias, const float* k_bias, const float* v_bias, int64_t num_tokens,
                                   int heads, int kv_heads, int dim, int vdim, int rot_dims, int adjacent, int norm_values,
                                   float eps, int qk_norm, const float* q_head_scale, float q_temp_coef, int q_temp_every,
                                   const void* v_first, int64_t vf_stride, const float* v_mix, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0);
  SP_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(q && k && v && kpool && vpool && positions && loc && (freq || rot_dims == 0));
  SP_CHECK_ARG(q_stride >= (int64_t)heads * dim && k_stride >= (int64_t)kv_heads * dim && v_stride >= (int64_t)kv_heads * vdim);
  SP_CHECK_ARG(kp_stride >= (int64_t)kv_heads * dim && vp_stride >= (int64_t)kv_heads * vdim);
  SP_CHECK_ARG(q_temp_every >= 0 && (!v_first || (v_mix && vf_stride >= (int64_t)kv_heads * vdim)));
  if (qk_norm || q_head_scale || q_temp_every > 0 || v_first) {      // the wave-per-head form
    if (dim > 64 * kStorePerLane || vdim > 64 * kStorePerLane) return SP_ERR_UNSUPPORTED;
    SP_DISPATCH_DTYPE(dtype, (qkv_norm_store_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                                 q, q_stride, k, k_stride, v, v_stride, kpool, kp_stride, vpool, vp_stride, positions, loc,
                                 freq, mag, q_bias, k_bias, v_bias, heads, kv_heads, dim, vdim, rot_dims, adjacent,
                                 norm_values, eps, qk_norm, q_head_scale, q_temp_coef, q_temp_every, v_first, vf_stride,
                                 v_mix)));
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  SP_DISPATCH_DTYPE(dtype, (qkv_rotary_store_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               q, q_stride, k, k_stride, v, v_stride, kpool, kp_stride, vpool, vp_stride, positions, loc,
                               freq, mag, q_bias, k_bias, v_bias, heads, kv_heads, dim, vdim, rot_dims, adjacent, norm_values,
                               eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_pool_blocks(void* kpooled, void* vpooled, const void* kpool, const void* vpool, int64_t kp_stride,
                              int64_t vp_stride, const int32_t* req_to_token, int64_t table_stride, int64_t num_tokens,
                              int key_width, int value_width, int block, SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && key_width > 0 && value_width > 0 && block > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(kpooled && vpooled && kpool && vpool && req_to_token && req_pool_indices && seq_lens);
  SP_CHECK_ARG(kp_stride >= key_width && vp_stride >= value_width);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, (pool_blocks_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               kpooled, vpooled, kpool, vpool, kp_stride, vp_stride, req_to_token, table_stride, s, key_width,
                               value_width, block)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_window_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kpool,
                                   const void* vpool, const void* kpooled, const void* vpooled, int64_t kp_stride,
                                   int64_t vp_stride, const int32_t* req_to_token, int64_t table_stride,
                                   int64_t num_tokens, int heads, int kv_heads, int dim, int vdim, int64_t window, int block,
                                   float scale, const float* sinks, float softcap, int sigmoid_weights,
                                   const float* head_bias, const void* gate, int64_t gate_stride, int matrix, SP_SEQ_PARAMS,
                                   int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(out && q && kpool && vpool && req_to_token && req_pool_indices && seq_lens);
  SP_CHECK_ARG((kpooled && vpooled) || block <= 0 || window <= 0);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
  SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  SP_CHECK_ARG(q_stride >= (int64_t)heads * dim && out_stride >= (int64_t)heads * vdim);
  SP_CHECK_ARG(kp_stride >= (int64_t)kv_heads * dim && vp_stride >= (int64_t)kv_heads * vdim);
  SP_CHECK_ARG(!gate || gate_stride >= (int64_t)heads * vdim);
  SP_CHECK_ARG(!sigmoid_weights || !sinks);
  if (vdim > 64 * kMaxPerLane) return SP_ERR_UNSUPPORTED;
  const int nw = extend_seq_lens ? 4 : 16;       // waves per (token, head): see the kernel
  const size_t lds = ((size_t)dim + 64 * nw + (size_t)nw * vdim + 2 * nw) * sizeof(float);
  if (lds > 64 * 1024) return SP_ERR_UNSUPPORTED;
  SEQ_BATCH(s);
  // portions of prompts in 16-bit types: the matrix-core kernel where its tile shapes and 16-byte row loads apply
  const bool al16 = (((uintptr_t)q | (uintptr_t)kpool | (uintptr_t)vpool | (uintptr_t)kpooled | (uintptr_t)vpooled) & 15) == 0 &&
                    ((uintptr_t)out & 7) == 0;
  if (matrix && extend_seq_lens && num_tokens > batch_size && (dtype == SP_BF16 || dtype == SP_F16) && (dim == 64 || dim == 128) &&
      (vdim == 64 || vdim == 128) && al16 && q_stride % 8 == 0 && kp_stride % 8 == 0 && vp_stride % 8 == 0 && out_stride % 4 == 0 &&
      (!gate || (((uintptr_t)gate & 7) == 0 && gate_stride % 4 == 0))) {
    const dim3 mgrid((unsigned)((num_tokens + 15) / 16 + batch_size), (unsigned)kv_heads);
#define SP_WM2(T, DS, DT, SG)                                                                                            \
  window_attention_mfma_kernel<T, DS, DT, SG><<<mgrid, 256, 0, (hipStream_t)stream>>>(                                     \
      out, out_stride, q, q_stride, kpool, vpool, kpooled, vpooled, kp_stride, vp_stride, req_to_token, table_stride, s, heads, \
      kv_heads, window, block, scale, sinks, softcap, head_bias, gate, gate_stride)
#define SP_WM(T, DS, DT)                    \
  do {                                      \
    if (sigmoid_weights) SP_WM2(T, DS, DT, true); \
    else SP_WM2(T, DS, DT, false);          \
  } while (0)
#define SP_WM_SHAPES(T)                                   \
  do {                                                    \
    if (dim == 64 && vdim == 64) SP_WM(T, 2, 4);          \
    else if (dim == 64) SP_WM(T, 2, 8);                   \
    else if (vdim == 64) SP_WM(T, 4, 4);                  \
    else SP_WM(T, 4, 8);                                  \
  } while (0)
    if (dtype == SP_BF16) SP_WM_SHAPES(bf16_tag);
    else SP_WM_SHAPES(f16_tag);
#undef SP_WM_SHAPES
#undef SP_WM
#undef SP_WM2
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  const dim3 grid((unsigned)num_tokens, (unsigned)heads);
  const int vecn = dtype == SP_F32 ? 4 : 8;
  const bool vec = dim % vecn == 0 && kp_stride % vecn == 0 && ((uintptr_t)kpool & 15) == 0 &&
                   (!kpooled || ((uintptr_t)kpooled & 15) == 0);
#define SP_WA(V, SG)                                                                                                   \
  SP_DISPATCH_DTYPE(dtype, (window_attention_kernel<Tag, V, SG><<<grid, 64 * nw, lds, (hipStream_t)stream>>>(           \
                               out, out_stride, q, q_stride, kpool, vpool, kpooled, vpooled, kp_stride, vp_stride,      \
                               req_to_token, table_stride, s, heads, kv_heads, dim, vdim, window, block, scale, sinks,  \
                               softcap, head_bias, gate, gate_stride)))
  if (vec && sigmoid_weights) SP_WA(true, true);
  else if (vec) SP_WA(true, false);
  else if (sigmoid_weights) SP_WA(false, true);
  else SP_WA(false, false);
#undef SP_WA
  SP_LAUNCH_CHECK();
  return SP_OK;
}
