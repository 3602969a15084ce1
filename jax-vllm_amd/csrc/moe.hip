// Routed experts: choice of experts per token, rows grouped by expert on the device, and the two
// grouped matrix products of gated experts.  Nothing here returns to the host: a step's routing is
// known only on the device, so every launch is sized by upper bounds and blocks without work leave.
//
//   route:   z = router logits (float, plus an optional bias per expert) -> the `top` largest per token
//            (lowest index among equals), weight = sigmoid(z), or the softmax over the chosen logits alone, or
//            ("sigmoid_normed") the largest sigmoid(z) + correction chosen, weight = sigmoid(z) over the sum of the
//            chosen sigmoids (+ 1e-20) times a constant
//   group:   entry s = token * top + kk  ->  position in a list ordered by expert; tiles of MOE_TM rows
//            that never straddle two experts
//   gate/up: z[pos] = act(w g) * (w u),  g = Wg[e] x[token], u = Wu[e] x[token]      (w = the entry's weight
//            when it scales the expert's INPUT: w (W x) = W (w x); else 1)
//   down:    y[kk][token] = (Wd[e] z[pos]) * (w if it scales the OUTPUT else 1)        float
// The order of rows inside an expert's group depends on timing; no result does: every output row is a
// sum over the inner size in ascending order, alone.
#include "common.h"

#define MOE_TM 64
#define MOE_TN 64
#define MOE_BK 16

// The `top` largest of a token's logits, lowest index among equals: the lanes of a wave scan the token's
// logits (a copy in LDS), the wave agrees on the best, and the lane that scans the chosen expert takes it out.
#define MOE_SCORE_SIGMOID 0          // weight = sigmoid(logit)
#define MOE_SCORE_SOFTMAX_CHOSEN 1   // weight = exp(logit) / sum of exp over the token's chosen logits
#define MOE_SCORE_SIGMOID_NORMED 2   // chosen by sigmoid(logit) + correction; weight = sigmoid(logit) / (sum over the chosen + 1e-20) * scale
__device__ __forceinline__ void moe_pick(float* zt, int experts, int top, int lane, int* ids, float* weights,
                                         int score, const float* __restrict__ correction = nullptr,
                                         float weight_scale = 1.f) {
  const bool normed = score == MOE_SCORE_SIGMOID_NORMED;
  for (int kk = 0; kk < top; ++kk) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < experts; e += JV_WAVE) {
      float v = zt[e];
      // an expert already taken holds -inf and stays out; the others compete with their corrected sigmoid
      if (normed && v != -INFINITY) v = 1.f / (1.f + expf(-v)) + (correction ? correction[e] : 0.f);
      if (v > bv || (bi == 0x7fffffff && v == v)) { bv = v; bi = e; }
    }
#pragma unroll
    for (int o = JV_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, JV_WAVE);
      const int oi = __shfl_xor(bi, o, JV_WAVE);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) { bi = kk; bv = __builtin_nanf(""); }      // a row of NaN: some expert, the NaN shows in the output
    if (lane == 0) {
      ids[kk] = bi;
      const float z = normed ? zt[bi] : bv;          // the logit itself: the correction takes part in the choice only
      weights[kk] = score == MOE_SCORE_SOFTMAX_CHOSEN ? bv : 1.f / (1.f + expf(-z));
    }
    if ((bi & (JV_WAVE - 1)) == lane) zt[bi] = -INFINITY;
  }
  if (score == MOE_SCORE_SOFTMAX_CHOSEN && lane == 0) {
    // the chosen logits came in descending order: the first is their maximum; sums in that order
    const float m = weights[0];
    float sum = 0.f;
    for (int kk = 0; kk < top; ++kk) {
      const float p = expf(weights[kk] - m);
      weights[kk] = p;
      sum += p;
    }
    const float inv = 1.f / sum;
    for (int kk = 0; kk < top; ++kk) weights[kk] *= inv;
  }
  if (normed && lane == 0) {
    float sum = 0.f;
    for (int kk = 0; kk < top; ++kk) sum += weights[kk];
    const float f = weight_scale / (sum + 1e-20f);
    for (int kk = 0; kk < top; ++kk) weights[kk] *= f;
  }
}

// a wave per token, 4 tokens a block
__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ logits, const float* __restrict__ bias, int n, int experts, int top,
                 int score, int* __restrict__ ids, float* __restrict__ weights, const float* __restrict__ correction,
                 float weight_scale) {
  extern __shared__ float zs[];      // [4][experts]
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  const long long t = (long long)blockIdx.x * 4 + wid;
  if (t >= n) return;
  float* zt = zs + wid * experts;
  for (int e = lane; e < experts; e += JV_WAVE) zt[e] = logits[t * experts + e] + (bias ? bias[e] : 0.f);
  moe_pick(zt, experts, top, lane, ids + t * top, weights + t * top, score, correction, weight_scale);
}

// Router and choice in one launch: a block takes up to MOE_RT tokens, their rows in LDS as floats; a wave per
// expert (in turns) reads the expert's router row once and sums its products with every token of the block
// lane by lane and then across the wave: float logits whatever the activation type, the same order of
// additions whatever the batch.  Then a wave per token picks the `top` largest, lowest index among equals.
// logits_out (may be null) [n, experts].
#define MOE_RT 8
template <typename T>
__global__ void __launch_bounds__(1024)
moe_router_kernel(const T* __restrict__ x, const T* __restrict__ W, const float* __restrict__ bias, int n, int hidden,
                  int experts, int top, int tb, int score, int* __restrict__ ids, float* __restrict__ weights,
                  float* __restrict__ logits_out, const float* __restrict__ correction, float weight_scale) {
  extern __shared__ float rs[];      // x [tb][hidden] | z [tb][experts]
  float* xs = rs;
  float* z = rs + tb * hidden;
  const long long t0 = (long long)blockIdx.x * tb;
  const int nt = (int)min((long long)tb, n - t0);
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE, nw = blockDim.x / JV_WAVE;
  for (int i = threadIdx.x; i < tb * hidden; i += blockDim.x) {
    const int t = i / hidden;
    xs[i] = t < nt ? to_f32(x[t0 * hidden + i]) : 0.f;
  }
  __syncthreads();
  for (int e = wid; e < experts; e += nw) {
    const T* w = W + (long long)e * hidden;
    float acc[MOE_RT];
#pragma unroll
    for (int t = 0; t < MOE_RT; ++t) acc[t] = 0.f;
    // eight loads of the router row are asked for before their products: a wave's time here is its chain of loads
    for (int c0 = lane; c0 < hidden; c0 += 8 * JV_WAVE) {
      float wv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int c = c0 + u * JV_WAVE;
        wv[u] = to_f32(w[c < hidden ? c : lane]);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int c = c0 + u * JV_WAVE;
        if (c < hidden) {
#pragma unroll
          for (int t = 0; t < MOE_RT; ++t)
            if (t < tb) acc[t] = fmaf(xs[t * hidden + c], wv[u], acc[t]);
        }
      }
    }
#pragma unroll
    for (int t = 0; t < MOE_RT; ++t) {
      if (t >= nt) continue;
      const float v = wave_sum(acc[t]) + (bias ? bias[e] : 0.f);
      if (lane == 0) {
        z[t * experts + e] = v;
        if (logits_out) logits_out[(t0 + t) * experts + e] = v;
      }
    }
  }
  __syncthreads();
  for (int t = wid; t < nt; t += nw)
    moe_pick(z + t * experts, experts, top, lane, ids + (t0 + t) * top, weights + (t0 + t) * top, score, correction,
             weight_scale);
}

// One block.  meta: [0] number of tiles; offsets [experts + 1]; tile_expert / tile_row0 [max_tiles];
// order [entries]: entry index at each position; rank [entries] scratch.  A tile has tile_rows rows.
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int* __restrict__ ids, int entries, int experts, int tile_rows, int* __restrict__ meta,
                 int* __restrict__ offsets, int* __restrict__ tile_expert, int* __restrict__ tile_row0,
                 int* __restrict__ order, int* __restrict__ rank) {
  extern __shared__ int sh[];      // count [experts] | start [experts + 1] | first tile [experts + 1]
  int* count = sh;
  int* start = sh + experts;
  int* tile0 = start + experts + 1;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int s = threadIdx.x; s < entries; s += blockDim.x) rank[s] = atomicAdd(&count[ids[s]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      start[e] = at;
      tile0[e] = tiles;
      at += count[e];
      tiles += (count[e] + tile_rows - 1) / tile_rows;
    }
    start[experts] = at;
    tile0[experts] = tiles;
    meta[0] = tiles;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= experts; e += blockDim.x) offsets[e] = start[e];
  for (int e = threadIdx.x; e < experts; e += blockDim.x)
    for (int i = tile0[e]; i < tile0[e + 1]; ++i) {
      tile_expert[i] = e;
      tile_row0[i] = start[e] + (i - tile0[e]) * tile_rows;
    }
  for (int s = threadIdx.x; s < entries; s += blockDim.x) order[start[ids[s]] + rank[s]] = s;
}

// grid (max tiles, column tiles of the expert width).  x [tokens, hidden]; Wg, Wu [experts, ff, hidden];
// z [entries, ff] by position.
template <typename T>
__global__ void __launch_bounds__(256)
moe_gate_up_kernel(T* __restrict__ z, const T* __restrict__ x, const T* __restrict__ Wg, const T* __restrict__ Wu,
                   const int* __restrict__ meta, const int* __restrict__ offsets, const int* __restrict__ tile_expert,
                   const int* __restrict__ tile_row0, const int* __restrict__ order, const float* __restrict__ weights,
                   int top, int hidden, int ff, int act, int scale_input) {
  if ((int)blockIdx.x >= meta[0]) return;
  __shared__ float As[MOE_BK][MOE_TM + 4];
  __shared__ float Gs[MOE_BK][MOE_TN + 4];
  __shared__ float Us[MOE_BK][MOE_TN + 4];
  __shared__ int tok[MOE_TM];
  __shared__ float wgt[MOE_TM];
  const int e = tile_expert[blockIdx.x], row0 = tile_row0[blockIdx.x];
  const int rows = min(MOE_TM, offsets[e + 1] - row0);
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.y * MOE_TN;
  if (tid < MOE_TM) {
    const int s = tid < rows ? order[row0 + tid] : -1;
    tok[tid] = s < 0 ? -1 : s / top;
    wgt[tid] = (s < 0 || !scale_input) ? 1.f : weights[s];
  }
  __syncthreads();
  const T* G = Wg + (long long)e * ff * hidden;
  const T* U = Wu + (long long)e * ff * hidden;
  float ag[4][4] = {}, au[4][4] = {};
  for (int k0 = 0; k0 < hidden; k0 += MOE_BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = tid + q * 256;
      const int r = idx >> 4, kk = idx & 15, k = k0 + kk;
      const int tk = tok[r], wn = n0 + r;
      As[kk][r] = (tk >= 0 && k < hidden) ? to_f32(x[(long long)tk * hidden + k]) : 0.f;
      const bool in = wn < ff && k < hidden;
      Gs[kk][r] = in ? to_f32(G[(long long)wn * hidden + k]) : 0.f;
      Us[kk][r] = in ? to_f32(U[(long long)wn * hidden + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < MOE_BK; ++kk) {
      float a[4], g[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) { g[j] = Gs[kk][tx * 4 + j]; u[j] = Us[kk][tx * 4 + j]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ag[i][j] = fmaf(a[i], g[j], ag[i][j]);
          au[i][j] = fmaf(a[i], u[j], au[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= rows) continue;
    const float w = wgt[m];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < ff) z[(long long)(row0 + m) * ff + n] = from_f32<T>(jv_gated(act, ag[i][j] * w, au[i][j] * w));
    }
  }
}

// grid (max tiles, column tiles of hidden).  z [entries, ff] by position; Wd [experts, hidden, ff];
// y [top, tokens, hidden] float.
template <typename T>
__global__ void __launch_bounds__(256)
moe_down_kernel(float* __restrict__ y, const T* __restrict__ z, const T* __restrict__ Wd, const int* __restrict__ meta,
                const int* __restrict__ offsets, const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
                const int* __restrict__ order, const float* __restrict__ weights, int top, int n_tokens, int hidden,
                int ff, int scale_output) {
  if ((int)blockIdx.x >= meta[0]) return;
  __shared__ float As[MOE_BK][MOE_TM + 4];
  __shared__ float Ws[MOE_BK][MOE_TN + 4];
  __shared__ int ent[MOE_TM];
  const int e = tile_expert[blockIdx.x], row0 = tile_row0[blockIdx.x];
  const int rows = min(MOE_TM, offsets[e + 1] - row0);
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.y * MOE_TN;
  if (tid < MOE_TM) ent[tid] = tid < rows ? order[row0 + tid] : -1;
  __syncthreads();
  const T* W = Wd + (long long)e * hidden * ff;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < ff; k0 += MOE_BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = tid + q * 256;
      const int r = idx >> 4, kk = idx & 15, k = k0 + kk;
      const int wn = n0 + r;
      As[kk][r] = (r < rows && k < ff) ? to_f32(z[(long long)(row0 + r) * ff + k]) : 0.f;
      Ws[kk][r] = (wn < hidden && k < ff) ? to_f32(W[(long long)wn * ff + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < MOE_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= rows) continue;
    const int s = ent[m];
    const int token = s / top, kk = s - token * top;
    const float w = scale_output ? weights[s] : 1.f;
    float* o = y + ((long long)kk * n_tokens + token) * hidden;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < hidden) o[n] = acc[i][j] * w;
    }
  }
}

// A share of every token that carries a gate of the token's own: out[t][c] = float(y[t][c]) * sigmoid(g[t * ldg])
// (a shared expert that joins the chosen experts' float stack under one number per token).
template <typename T>
__global__ void __launch_bounds__(256)
row_gate_kernel(float* __restrict__ out, const T* __restrict__ y, const T* __restrict__ g, long long ldg, long long n,
                int hidden) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * hidden) return;
  const long long t = i / hidden;
  out[i] = to_f32(y[i]) / (1.f + expf(-to_f32(g[t * ldg])));
}

// The same with four columns a lane, where the width and the addresses allow it.
template <typename T>
__global__ void __launch_bounds__(256)
row_gate_vec_kernel(float* __restrict__ out, const T* __restrict__ y, const T* __restrict__ g, long long ldg, long long n,
                    int hidden) {
  typedef T t4 __attribute__((ext_vector_type(4)));
  const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n * hidden) return;
  const long long t = i / hidden;
  const float gate = 1.f / (1.f + expf(-to_f32(g[t * ldg])));
  const t4 v = *(const t4*)(y + i);
  *(float4*)(out + i) = float4{to_f32(v[0]) * gate, to_f32(v[1]) * gate, to_f32(v[2]) * gate, to_f32(v[3]) * gate};
}

extern "C" int jv_moe_tile_rows() { return MOE_TM; }

extern "C" int jv_moe_route(const float* logits, const float* bias, int n, int experts, int top, int score, int* ids,
                            float* weights, const float* correction, float weight_scale, void* stream) {
  if (n <= 0) return 0;
  if (experts <= 0 || top <= 0 || top > experts || score < 0 || score > MOE_SCORE_SIGMOID_NORMED)
    return (int)hipErrorInvalidValue;
  if (experts > 3840) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_route_kernel, dim3((n + 3) / 4), dim3(256), 4 * experts * sizeof(float), (hipStream_t)stream,
                     logits, bias, n, experts, top, score, ids, weights, correction, weight_scale);
  return JV_LAUNCH_CHECK();
}

extern "C" int jv_moe_group(const int* ids, int entries, int experts, int tile_rows, int* meta, int* offsets,
                            int* tile_expert, int* tile_row0, int* order, int* rank, void* stream) {
  if (entries <= 0) return 0;
  if (experts <= 0 || experts > 4096 || tile_rows <= 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), (3 * experts + 2) * sizeof(int), (hipStream_t)stream, ids,
                     entries, experts, tile_rows, meta, offsets, tile_expert, tile_row0, order, rank);
  return JV_LAUNCH_CHECK();
}

#define DEFINE_MOE(SUF, T)                                                                                        \
  extern "C" int jv_moe_router_##SUF(const void* x, const void* W, const float* bias, int n, int hidden,          \
                                     int experts, int top, int score, int* ids, float* weights,                   \
                                     float* logits_out, const float* correction, float weight_scale,              \
                                     void* stream) {                                                              \
    if (n <= 0) return 0;                                                                                         \
    if (experts <= 0 || top <= 0 || top > experts || hidden <= 0 || (hidden + experts) > 15000 || score < 0 ||    \
        score > MOE_SCORE_SIGMOID_NORMED)                                                                         \
      return (int)hipErrorInvalidValue;                                                                           \
    int tb = 15000 / (hidden + experts);             /* tokens of a block: their rows and logits in 60 KB */      \
    tb = tb > MOE_RT ? MOE_RT : tb;                                                                               \
    while (tb > 1 && (n + tb - 1) / tb < 128) --tb;  /* few tokens: more blocks rather than rows sharing a read */ \
    hipLaunchKernelGGL(moe_router_kernel<T>, dim3((n + tb - 1) / tb), dim3(1024),                                  \
                       (size_t)tb * (hidden + experts) * sizeof(float), (hipStream_t)stream, (const T*)x,         \
                       (const T*)W, bias, n, hidden, experts, top, tb, score, ids, weights, logits_out,           \
                       correction, weight_scale);                                                                 \
    return JV_LAUNCH_CHECK();                                                                                     \
  }                                                                                                               \
  extern "C" int jv_row_gate_##SUF(float* out, const void* y, const void* g, long long ldg, long long n,         \
                                   int hidden, void* stream) {                                                    \
    if (n <= 0 || hidden <= 0) return 0;                                                                          \
    if ((n * hidden + 255) / 256 > 0x7fffffffll) return (int)hipErrorInvalidValue;                                \
    if (hidden % 4 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)y % (4 * sizeof(T)) == 0) {                     \
      hipLaunchKernelGGL(row_gate_vec_kernel<T>, dim3((unsigned)((n * hidden / 4 + 255) / 256)), dim3(256), 0,    \
                         (hipStream_t)stream, out, (const T*)y, (const T*)g, ldg, n, hidden);                     \
      return JV_LAUNCH_CHECK();                                                                                   \
    }                                                                                                             \
    hipLaunchKernelGGL(row_gate_kernel<T>, dim3((unsigned)((n * hidden + 255) / 256)), dim3(256), 0,              \
                       (hipStream_t)stream, out, (const T*)y, (const T*)g, ldg, n, hidden);                       \
    return JV_LAUNCH_CHECK();                                                                                     \
  }                                                                                                               \
  extern "C" int jv_moe_gate_up_##SUF(void* z, const void* x, const void* Wg, const void* Wu, const int* meta,    \
                                      const int* offsets, const int* tile_expert, const int* tile_row0,           \
                                      const int* order, const float* weights, int max_tiles, int top, int hidden, \
                                      int ff, int act, int scale_input, void* stream) {                           \
    if (max_tiles <= 0 || ff <= 0) return 0;                                                                      \
    if (!jv_act_known(act) || (ff + MOE_TN - 1) / MOE_TN > 65535) return (int)hipErrorInvalidValue;               \
    hipLaunchKernelGGL(moe_gate_up_kernel<T>, dim3(max_tiles, (ff + MOE_TN - 1) / MOE_TN), dim3(256), 0,          \
                       (hipStream_t)stream, (T*)z, (const T*)x, (const T*)Wg, (const T*)Wu, meta, offsets,        \
                       tile_expert, tile_row0, order, weights, top, hidden, ff, act, scale_input);                \
    return JV_LAUNCH_CHECK();                                                                                     \
  }                                                                                                               \
  extern "C" int jv_moe_down_##SUF(float* y, const void* z, const void* Wd, const int* meta, const int* offsets,  \
                                   const int* tile_expert, const int* tile_row0, const int* order,                \
                                   const float* weights, int max_tiles, int top, int n_tokens, int hidden,        \
                                   int ff, int scale_output, void* stream) {                                      \
    if (max_tiles <= 0 || hidden <= 0) return 0;                                                                  \
    if ((hidden + MOE_TN - 1) / MOE_TN > 65535) return (int)hipErrorInvalidValue;                                 \
    hipLaunchKernelGGL(moe_down_kernel<T>, dim3(max_tiles, (hidden + MOE_TN - 1) / MOE_TN), dim3(256), 0,         \
                       (hipStream_t)stream, y, (const T*)z, (const T*)Wd, meta, offsets, tile_expert, tile_row0,  \
                       order, weights, top, n_tokens, hidden, ff, scale_output);                                  \
    return JV_LAUNCH_CHECK();                                                                                     \
  }

DEFINE_MOE(bf16, bf16_t)
DEFINE_MOE(f32, float)
