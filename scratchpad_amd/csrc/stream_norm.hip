// fp32 residual stream of parallel-sublayer models:  x <- x + mixer(shift(h)) + ff(h),  h = x / rms(x) * w.
//   scaled embedding      x[t]  = embed[id[t]] * scale                                     (fp32)
//   norm + token shift    h[t]  = x[t] / sqrt(mean(x[t]^2) + eps) * w                      (what the feed-forward reads)
//                         hs[t] = h[t] + (h[t-1] - h[t]) * mu                              (what the mixer reads)
//                         h[-1] of a step's first row = the request's saved h (zeros at a sequence's first token)
//   saved h               state[slot] = h[the request's last row of this step]             (fp32, a launch of its own:
//                                                                                           every reader has finished)
//   sum                   x[t] += a[t] + b[t] + c[t]                                       (fp32; b, c optional)
// and of sequential-sublayer models that gate and norm a sublayer's RESULT before it joins the stream:
//   gated normed sum      y = a  or  (N(a) wa + N(b) wb) / 2;   y *= sigmoid(gate + gate_bias);   x += N(y) w;
//                         x += extra;   next = N(x) w_next      (N = division by the row's root mean square)
// and of sequential pre-norm models whose norm works in groups:
//   sum + group norm      x += a  or  x += (N(a) wa + N(b) wb) / 2  (or nothing);   next = GN(x) w_next, GN = every one of
//                         `groups` equal consecutive parts of the row divided by its own root mean square
// All arithmetic is fp32; h and hs are rounded once, to the projections' element type.
#include "seq_batch.h"

namespace sp {
namespace {

template <typename Tag>
__global__ void embed_scale_kernel(float* x, int64_t x_stride, const void* embed, const int64_t* ids, int width,
                                   int64_t vocab, float scale) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int i = threadIdx.x; i < width; i += blockDim.x) x[t * x_stride + i] = E::load(embed, id * width + i) * scale;
}

// one workgroup per row: the row's own norm and, for the shift, the previous row's (recomputed: two reads of a row
// are cheaper than a second launch and an fp32 copy of h)
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
norm_shift_kernel(void* out_h, void* out_hs, int64_t out_stride, const float* x, int64_t x_stride, const float* w,
                  const float* mu, const float* state, int64_t state_stride, SeqBatch s, int width, float eps) {
  typedef Elem<Tag> E;
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  const float* row = x + t * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += row[i] * row[i];
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  if (!out_hs) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) E::store(out_h, t * out_stride + i, row[i] * inv * w[i]);
    return;
  }
  int b;
  int64_t start, prefix;
  seq_of_token(s, t, b, start, prefix);
  const float* prow = nullptr;       // previous row of x (its norm is computed here)
  const float* saved = nullptr;      // or the saved h
  float pinv = 0.f;
  if (t > start) {
    prow = x + (t - 1) * x_stride;
    float ps = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) ps += prow[i] * prow[i];
    ps = block_sum(ps, red);
    pinv = 1.f / sqrtf(ps / (float)width + eps);
  } else if (prefix > 0) {
    saved = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float h = row[i] * inv * w[i];
    const float hp = prow ? prow[i] * pinv * w[i] : (saved ? saved[i] : 0.f);
    if (out_h) E::store(out_h, t * out_stride + i, h);
    E::store(out_hs, t * out_stride + i, h + (hp - h) * mu[i]);
  }
}

// state[slot of request b] = h[last row of b]
__global__ void __launch_bounds__(kBlock)
norm_save_kernel(float* state, int64_t state_stride, const float* x, int64_t x_stride, const float* w, SeqBatch s, int width,
                 float eps) {
  __shared__ float red[kBlock / 64];
  const int b = blockIdx.x;
  int64_t start, len, prefix;
  seq_span(s, b, start, len, prefix);
  if (len <= 0) return;
  const float* row = x + (start + len - 1) * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += row[i] * row[i];
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  float* dst = state + load_idx(s.req_pool_indices, b, s.idx64) * state_stride;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = row[i] * inv * w[i];
}

template <typename Tag>
__global__ void stream_add_kernel(float* x, int64_t x_stride, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                                  const void* c, int64_t c_stride, int width) {
  typedef Elem<Tag> E;
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float y = E::load(a, t * a_stride + i);
    if (b) y += E::load(b, t * b_stride + i);
    if (c) y += E::load(c, t * c_stride + i);
    x[t * x_stride + i] += y;
  }
}


// one workgroup per row; the row's y, then its new x, wait in LDS between the reductions (each thread reads back only what
// it wrote itself, so the reductions' barriers are the only ones)
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
gated_add_norm_kernel(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                      int64_t b_stride, const float* wb, const void* gate, int64_t gate_stride, const float* gate_bias,
                      const float* weight, const float* extra, int64_t extra_stride, void* out_next, int64_t next_stride,
                      const float* next_weight, int width, float eps) {
  typedef Elem<Tag> E;
  extern __shared__ float rowbuf[];
  __shared__ float red[kBlock / 64];
  const int64_t t = blockIdx.x;
  float ia = 1.f, ib = 0.f;
  if (b) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float u = E::load(a, t * a_stride + i), v = E::load(b, t * b_stride + i);
      sa += u * u;
      sb += v * v;
    }
    sa = block_sum(sa, red);
    sb = block_sum(sb, red);
    ia = 1.f / sqrtf(sa / (float)width + eps);
    ib = 1.f / sqrtf(sb / (float)width + eps);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float y = E::load(a, t * a_stride + i);
    if (b) y = 0.5f * (y * ia * wa[i] + E::load(b, t * b_stride + i) * ib * wb[i]);
    if (gate) y /= 1.f + expf(-(E::load(gate, t * gate_stride + i) + (gate_bias ? gate_bias[i] : 0.f)));
    rowbuf[i] = y;
    ss += y * y;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  float sx = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[t * x_stride + i] + rowbuf[i] * inv * weight[i];
    if (extra) v += extra[t * extra_stride + i];
    x[t * x_stride + i] = v;
    rowbuf[i] = v;
    sx += v * v;
  }
  if (!out_next) return;
  sx = block_sum(sx, red);
  const float invx = 1.f / sqrtf(sx / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) E::store(out_next, t * next_stride + i, rowbuf[i] * invx * next_weight[i]);
}

// The same on 16-byte vectors, for rows of NV x 256 vectors at most: a thread holds its part of the row in registers, every
// activation it needs (a, b, gate, x, extra) is loaded before the first reduction, and the three norms follow one another
// without a further pass over memory.
template <typename Tag, int NV>
__global__ void __launch_bounds__(kBlock)
gated_add_norm_vec_kernel(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                          int64_t b_stride, const float* wb, const void* gate, int64_t gate_stride, const float* gate_bias,
                          const float* weight, const float* extra, int64_t extra_stride, void* out_next, int64_t next_stride,
                          const float* next_weight, int width, float eps) {
  typedef Elem<Tag> E;
  constexpr int V = E::kVec;
  __shared__ float red[2 * (kBlock / 64)];
  const int64_t t = blockIdx.x;
  const int nvec = width / V;
  float ya[NV][V], yb[NV][V], yg[NV][V], xs[NV][V];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    const bool on = vi < nvec;
    const int64_t c = (int64_t)vi * V;
    if (on) {
      unpack16<Tag>(ld16((const char*)a + (t * a_stride + c) * E::kBytes), ya[u]);
      if (b) unpack16<Tag>(ld16((const char*)b + (t * b_stride + c) * E::kBytes), yb[u]);
      if (gate) unpack16<Tag>(ld16((const char*)gate + (t * gate_stride + c) * E::kBytes), yg[u]);
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        unpack16<f32_tag>(ld16(x + t * x_stride + c + 4 * q), xs[u] + 4 * q);
        if (extra) {
          float ex[4];
          unpack16<f32_tag>(ld16(extra + t * extra_stride + c + 4 * q), ex);
#pragma unroll
          for (int e = 0; e < 4; ++e) xs[u][4 * q + e] += ex[e];
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) ya[u][e] = yb[u][e] = yg[u][e] = xs[u][e] = 0.f;
    }
  }
  auto sum2 = [&](float& p, float& q) {           // two sums over the workgroup at once
    p = wave_sum(p);
    q = wave_sum(q);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) {
      red[2 * wave] = p;
      red[2 * wave + 1] = q;
    }
    __syncthreads();
    p = q = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) {
      p += red[2 * w];
      q += red[2 * w + 1];
    }
  };
  auto row4 = [&](const float* w, int64_t c, float* f) { unpack16<f32_tag>(ld16(w + c), f); };
  if (b) {
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u)
#pragma unroll
      for (int e = 0; e < V; ++e) {
        sa += ya[u][e] * ya[u][e];
        sb += yb[u][e] * yb[u][e];
      }
    sum2(sa, sb);
    const float ia = 1.f / sqrtf(sa / (float)width + eps), ib = 1.f / sqrtf(sb / (float)width + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int vi = threadIdx.x + u * kBlock;
      if (vi < nvec) {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
          float fa[4], fb[4];
          row4(wa, (int64_t)vi * V + 4 * q, fa);
          row4(wb, (int64_t)vi * V + 4 * q, fb);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            ya[u][4 * q + e] = 0.5f * (ya[u][4 * q + e] * ia * fa[e] + yb[u][4 * q + e] * ib * fb[e]);
        }
      }
    }
  }
  float ss = 0.f, unused = 0.f;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    if (gate && vi < nvec) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        float gb[4] = {0.f, 0.f, 0.f, 0.f};
        if (gate_bias) row4(gate_bias, (int64_t)vi * V + 4 * q, gb);
#pragma unroll
        for (int e = 0; e < 4; ++e) ya[u][4 * q + e] /= 1.f + expf(-(yg[u][4 * q + e] + gb[e]));
      }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) ss += ya[u][e] * ya[u][e];
  }
  sum2(ss, unused);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  float sx = 0.f;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    if (vi < nvec) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        float fw[4];
        row4(weight, (int64_t)vi * V + 4 * q, fw);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          xs[u][4 * q + e] += ya[u][4 * q + e] * inv * fw[e];      // (the pass's added rows joined x when it was loaded)
        }
        st16(x + t * x_stride + (int64_t)vi * V + 4 * q, pack16<f32_tag>(xs[u] + 4 * q));
      }
#pragma unroll
      for (int e = 0; e < V; ++e) sx += xs[u][e] * xs[u][e];
    }
  }
  if (!out_next) return;
  sum2(sx, unused);
  const float invx = 1.f / sqrtf(sx / (float)width + eps);
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    if (vi < nvec) {
      float o[V];
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        float fw[4];
        row4(next_weight, (int64_t)vi * V + 4 * q, fw);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[4 * q + e] = xs[u][4 * q + e] * invx * fw[e];
      }
      st16((char*)out_next + (t * next_stride + (int64_t)vi * V) * E::kBytes, pack16<Tag>(o));
    }
  }
}

// one workgroup per row: the row's new x waits in LDS; wave w then forms the norm of the groups w, w + waves, ...
template <typename Tag>
__global__ void __launch_bounds__(kBlock)
add_group_norm_kernel(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                      int64_t b_stride, const float* wb, void* out_next, int64_t next_stride, const float* next_weight,
                      int width, int groups, float eps) {
  typedef Elem<Tag> E;
  extern __shared__ float rowbuf[];                  // [width] the row, then [groups] the inverse roots
  __shared__ float red[kBlock / 64];
  float* ginv = rowbuf + width;
  const int64_t t = blockIdx.x;
  float ia = 1.f, ib = 0.f;
  if (b) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float u = E::load(a, t * a_stride + i), v = E::load(b, t * b_stride + i);
      sa += u * u;
      sb += v * v;
    }
    sa = block_sum(sa, red);
    sb = block_sum(sb, red);
    ia = 1.f / sqrtf(sa / (float)width + eps);
    ib = 1.f / sqrtf(sb / (float)width + eps);
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[t * x_stride + i];
    if (a) {
      float y = E::load(a, t * a_stride + i);
      if (b) y = 0.5f * (y * ia * wa[i] + E::load(b, t * b_stride + i) * ib * wb[i]);
      v += y;
      x[t * x_stride + i] = v;
    }
    rowbuf[i] = v;
  }
  if (!out_next) return;
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, per = width / groups;
  for (int g = wave; g < groups; g += (int)(blockDim.x >> 6)) {
    float ss = 0.f;
    for (int i = lane; i < per; i += 64) ss += rowbuf[g * per + i] * rowbuf[g * per + i];
    ss = wave_sum(ss);
    if (lane == 0) ginv[g] = 1.f / sqrtf(ss / (float)per + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    E::store(out_next, t * next_stride + i, rowbuf[i] * ginv[i / per] * next_weight[i]);
}

// The same on 16-byte vectors, for rows of NV x 256 vectors at most whose groups are whole vectors: a thread holds its part
// of the row in registers; the vectors' sums of squares meet in LDS, where a wave per group adds them in a fixed order.
template <typename Tag, int NV>
__global__ void __launch_bounds__(kBlock)
add_group_norm_vec_kernel(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                          int64_t b_stride, const float* wb, void* out_next, int64_t next_stride, const float* next_weight,
                          int width, int groups, float eps) {
  typedef Elem<Tag> E;
  constexpr int V = E::kVec;
  __shared__ float red[2 * (kBlock / 64)];
  __shared__ float vsq[NV * kBlock];
  __shared__ float ginv[64];
  const int64_t t = blockIdx.x;
  const int nvec = width / V;
  float ya[NV][V], yb[NV][V], xs[NV][V];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    const int64_t c = (int64_t)vi * V;
    if (vi < nvec) {
      if (a) unpack16<Tag>(ld16((const char*)a + (t * a_stride + c) * E::kBytes), ya[u]);
      if (b) unpack16<Tag>(ld16((const char*)b + (t * b_stride + c) * E::kBytes), yb[u]);
#pragma unroll
      for (int q = 0; q < V / 4; ++q) unpack16<f32_tag>(ld16(x + t * x_stride + c + 4 * q), xs[u] + 4 * q);
    }
    if (vi >= nvec || !a) {
#pragma unroll
      for (int e = 0; e < V; ++e) ya[u][e] = 0.f;
    }
    if (vi >= nvec || !b) {
#pragma unroll
      for (int e = 0; e < V; ++e) yb[u][e] = 0.f;
    }
    if (vi >= nvec) {
#pragma unroll
      for (int e = 0; e < V; ++e) xs[u][e] = 0.f;
    }
  }
  auto row4 = [&](const float* w, int64_t c, float* f) { unpack16<f32_tag>(ld16(w + c), f); };
  if (b) {
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u)
#pragma unroll
      for (int e = 0; e < V; ++e) {
        sa += ya[u][e] * ya[u][e];
        sb += yb[u][e] * yb[u][e];
      }
    sa = wave_sum(sa);
    sb = wave_sum(sb);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
      red[2 * wave] = sa;
      red[2 * wave + 1] = sb;
    }
    __syncthreads();
    sa = sb = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) {
      sa += red[2 * w];
      sb += red[2 * w + 1];
    }
    const float ia = 1.f / sqrtf(sa / (float)width + eps), ib = 1.f / sqrtf(sb / (float)width + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int vi = threadIdx.x + u * kBlock;
      if (vi < nvec) {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
          float fa[4], fb[4];
          row4(wa, (int64_t)vi * V + 4 * q, fa);
          row4(wb, (int64_t)vi * V + 4 * q, fb);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            ya[u][4 * q + e] = 0.5f * (ya[u][4 * q + e] * ia * fa[e] + yb[u][4 * q + e] * ib * fb[e]);
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      xs[u][e] += ya[u][e];
      sq += xs[u][e] * xs[u][e];
    }
    if (vi < nvec) {
      vsq[vi] = sq;
      if (a) {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) st16(x + t * x_stride + (int64_t)vi * V + 4 * q, pack16<f32_tag>(xs[u] + 4 * q));
      }
    }
  }
  if (!out_next) return;
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, pv = nvec / groups;      // vectors per group
  for (int g = wave; g < groups; g += kBlock / 64) {
    float ss = 0.f;
    for (int i = lane; i < pv; i += 64) ss += vsq[g * pv + i];
    ss = wave_sum(ss);
    if (lane == 0) ginv[g] = 1.f / sqrtf(ss / (float)(pv * V) + eps);
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int vi = threadIdx.x + u * kBlock;
    if (vi < nvec) {
      const float inv = ginv[vi / pv];
      float o[V];
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        float fw[4];
        row4(next_weight, (int64_t)vi * V + 4 * q, fw);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[4 * q + e] = xs[u][4 * q + e] * inv * fw[e];
      }
      st16((char*)out_next + (t * next_stride + (int64_t)vi * V) * E::kBytes, pack16<Tag>(o));
    }
  }
}

}  // namespace
}  // namespace sp

using namespace sp;

extern "C" int sp_embed_scale(float* x, int64_t x_stride, const void* embed, const int64_t* ids, int64_t num_tokens,
                              int width, int64_t vocab, float scale, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && vocab > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && embed && ids && x_stride >= width);
  SP_DISPATCH_DTYPE(dtype, (embed_scale_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               x, x_stride, embed, ids, width, vocab, scale)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_norm_shift(void* out_h, void* out_hs, int64_t out_stride, const float* x, int64_t x_stride,
                             const float* weight, const float* mu, const float* state, int64_t state_stride,
                             int64_t num_tokens, int width, float eps, SP_SEQ_PARAMS, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG((out_h || out_hs) && x && weight && x_stride >= width && out_stride >= width);
  if (out_hs) {
    SP_CHECK_ARG(mu && state && state_stride >= width && req_pool_indices && seq_lens);
    SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc && token_req));
    SP_CHECK_ARG(extend_seq_lens || num_tokens == batch_size);
  }
  SEQ_BATCH(s);
  SP_DISPATCH_DTYPE(dtype, (norm_shift_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               out_h, out_hs, out_stride, x, x_stride, weight, mu, state, state_stride, s, width, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_norm_save_last(float* state, int64_t state_stride, const float* x, int64_t x_stride, const float* weight,
                                 int width, float eps, SP_SEQ_PARAMS, void* stream) {
  SP_CHECK_ARG(batch_size >= 0 && width > 0);
  if (batch_size == 0) return SP_OK;
  SP_CHECK_ARG(state && x && weight && state_stride >= width && x_stride >= width && req_pool_indices && seq_lens);
  SP_CHECK_ARG(!extend_seq_lens || (extend_prefix_lens && extend_start_loc));
  SEQ_BATCH(s);
  norm_save_kernel<<<dim3((unsigned)batch_size), kBlock, 0, (hipStream_t)stream>>>(state, state_stride, x, x_stride, weight,
                                                                                  s, width, eps);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_stream_add(float* x, int64_t x_stride, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                             const void* c, int64_t c_stride, int64_t num_tokens, int width, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && a && x_stride >= width && a_stride >= width && (!b || b_stride >= width) && (!c || c_stride >= width));
  SP_DISPATCH_DTYPE(dtype, (stream_add_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>(
                               x, x_stride, a, a_stride, b, b_stride, c, c_stride, width)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_gated_add_norm(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                                 int64_t b_stride, const float* wb, const void* gate, int64_t gate_stride,
                                 const float* gate_bias, const float* weight, const float* extra, int64_t extra_stride,
                                 void* out_next, int64_t next_stride, const float* next_weight, int64_t num_tokens, int width,
                                 float eps, int dtype, void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && width <= 15360);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && a && weight && x_stride >= width && a_stride >= width);
  SP_CHECK_ARG(!b || (wa && wb && b_stride >= width));
  SP_CHECK_ARG(!gate || gate_stride >= width);
  SP_CHECK_ARG(!extra || extra_stride >= width);
  SP_CHECK_ARG(!out_next || (next_weight && next_stride >= width));
  // rows of 16-byte vectors that 256 threads hold in registers: the vector kernel; anything else: the scalar one
  const int vecn = dtype == SP_F32 ? 4 : 8, esize = dtype == SP_F32 ? 4 : 2;
  auto al = [&](const void* p, int64_t stride, int elem_bytes) {
    return !p || ((((uintptr_t)p) & 15) == 0 && (stride * elem_bytes) % 16 == 0);
  };
  const bool vec = width % vecn == 0 && width / vecn <= 4 * kBlock && al(x, x_stride, 4) && al(a, a_stride, esize) &&
                   al(b, b_stride, esize) && al(gate, gate_stride, esize) && al(extra, extra_stride, 4) &&
                   al(out_next, next_stride, esize) && al(weight, 0, 4) && al(wa, 0, 4) && al(wb, 0, 4) && al(gate_bias, 0, 4) &&
                   al(next_weight, 0, 4);
  if (vec) {
    const int nv = (width / vecn + kBlock - 1) / kBlock;
#define SP_GAN(NV)                                                                                                      \
  SP_DISPATCH_DTYPE(dtype, (gated_add_norm_vec_kernel<Tag, NV><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>( \
                               x, x_stride, a, a_stride, wa, b, b_stride, wb, gate, gate_stride, gate_bias, weight, extra,  \
                               extra_stride, out_next, next_stride, next_weight, width, eps)))
    if (nv <= 1) SP_GAN(1);
    else if (nv <= 2) SP_GAN(2);
    else SP_GAN(4);
#undef SP_GAN
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  SP_DISPATCH_DTYPE(dtype, (gated_add_norm_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock, (size_t)width * sizeof(float),
                                                          (hipStream_t)stream>>>(
                               x, x_stride, a, a_stride, wa, b, b_stride, wb, gate, gate_stride, gate_bias, weight, extra,
                               extra_stride, out_next, next_stride, next_weight, width, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_add_group_norm(float* x, int64_t x_stride, const void* a, int64_t a_stride, const float* wa, const void* b,
                                 int64_t b_stride, const float* wb, void* out_next, int64_t next_stride,
                                 const float* next_weight, int64_t num_tokens, int width, int groups, float eps, int dtype,
                                 void* stream) {
  SP_CHECK_ARG(num_tokens >= 0 && width > 0 && width <= 15360 && groups > 0 && groups <= 64 && width % groups == 0);
  if (num_tokens == 0) return SP_OK;
  SP_CHECK_ARG(x && x_stride >= width && (a || out_next));
  SP_CHECK_ARG(!a || a_stride >= width);
  SP_CHECK_ARG(!b || (a && wa && wb && b_stride >= width));
  SP_CHECK_ARG(!out_next || (next_weight && next_stride >= width));
  // rows of 16-byte vectors that 256 threads hold in registers, groups of whole vectors: the vector kernel
  const int vecn = dtype == SP_F32 ? 4 : 8, esize = dtype == SP_F32 ? 4 : 2;
  auto al = [&](const void* p, int64_t stride, int elem_bytes) {
    return !p || ((((uintptr_t)p) & 15) == 0 && (stride * elem_bytes) % 16 == 0);
  };
  if (width % vecn == 0 && (width / groups) % vecn == 0 && width / vecn <= 4 * kBlock && al(x, x_stride, 4) &&
      al(a, a_stride, esize) && al(b, b_stride, esize) && al(out_next, next_stride, esize) && al(wa, 0, 4) && al(wb, 0, 4) &&
      al(next_weight, 0, 4)) {
    const int nv = (width / vecn + kBlock - 1) / kBlock;
#define SP_AGN(NV)                                                                                                      \
  SP_DISPATCH_DTYPE(dtype, (add_group_norm_vec_kernel<Tag, NV><<<dim3((unsigned)num_tokens), kBlock, 0, (hipStream_t)stream>>>( \
                               x, x_stride, a, a_stride, wa, b, b_stride, wb, out_next, next_stride, next_weight, width, groups, \
                               eps)))
    if (nv <= 1) SP_AGN(1);
    else if (nv <= 2) SP_AGN(2);
    else SP_AGN(4);
#undef SP_AGN
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  SP_DISPATCH_DTYPE(dtype, (add_group_norm_kernel<Tag><<<dim3((unsigned)num_tokens), kBlock,
                                                          (size_t)(width + groups) * sizeof(float), (hipStream_t)stream>>>(
                               x, x_stride, a, a_stride, wa, b, b_stride, wb, out_next, next_stride, next_weight, width,
                               groups, eps)));
  SP_LAUNCH_CHECK();
  return SP_OK;
}
