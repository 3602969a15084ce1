// Attention over one cached latent per token: the kernels around the paged attention kernels.
//
// A token caches the vector e = [c (rank floats, normed) | k_rot (rot floats, rotated)] once, for all heads.
// Every head's unrotated key is U_k[h] c and its value U_v[h] c, so with q'[h] = U_k[h]^T q_plain[h]
//   score = q'[h] . c + q_rot[h] . k_rot        and        value = U_v[h] (sum_j p_j c_j):
// attention with ONE kv head of size rank + rot whose keys and values are the same cached vector (the last rot
// elements of the weighted sum are not used).  The cache holds e in the two layouts the attention kernels
// read: key pages [page][1][slot][E] and transposed value pages [page][1][E][slot].
#include "common.h"

// cos_sin[t, 0:half] = amp * cos(pos_t * inv_freq), cos_sin[t, half:2 half] = amp * sin(...): a rotation whose
// frequencies were rescaled for longer contexts also scales both by a constant.
__global__ void rope_table_amp_kernel(float* __restrict__ cos_sin, const int* __restrict__ positions,
                                      const float* __restrict__ inv_freq, int half, float amp) {
  const long long t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int p = threadIdx.x; p < half; p += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[p], &s, &c);
    cos_sin[t * 2 * half + p] = c * amp;
    cos_sin[t * 2 * half + half + p] = s * amp;
  }
}

extern "C" int jv_rope_table_amp(float* cos_sin, const int* positions, const float* inv_freq, int n_tokens,
                                 int half, float amp, void* stream) {
  if (n_tokens <= 0 || half <= 0) return 0;
  hipLaunchKernelGGL(rope_table_amp_kernel, dim3(n_tokens), dim3(half >= 128 ? 128 : 64), 0,
                     (hipStream_t)stream, cos_sin, positions, inv_freq, half, amp);
  return JV_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- what follows the down-projections
// proj[t] = [ q latent (q_rank) | kv latent (rank) | rotated key part (rot) | ... ] in the activation type.
//   cq[t]  = T( norm(q latent) * wq )
//   e[t]   = [ T( norm(kv latent) * wkv ) | rotate(key part) ]  -> key page and transposed value page of the
//            token's slot (slot_mapping[t] < 0: nothing is stored)
// rotate: element i < half pairs with i + half (half = rot_dims / 2), or (interleaved) element 2i with 2i + 1,
// both by the angle of frequency i; elements from rot_dims on pass.  q_rank may be 0 (queries that are projected
// directly: no query latent, cq null); the kv latent begins at column kv_off of the row.
// One block per token.
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ proj, long long ld, int q_rank, long long kv_off, int rank, int rot,
                      int rot_dims, int interleaved,
                      const float* __restrict__ wq, const float* __restrict__ wkv, float eps,
                      const float* __restrict__ cos_sin, const int* __restrict__ slot_mapping,
                      T* __restrict__ cq, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size) {
  __shared__ float red[32];
  const long long t = blockIdx.x;
  const T* x = proj + t * ld;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x) { const float v = to_f32(x[c]); sq += v * v; }
  for (int c = threadIdx.x; c < rank; c += blockDim.x) { const float v = to_f32(x[kv_off + c]); sk += v * v; }
  if (q_rank) sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float inv_q = q_rank ? rsqrtf(sq / (float)q_rank + eps) : 0.f, inv_k = rsqrtf(sk / (float)rank + eps);
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x)
    cq[t * q_rank + c] = from_f32<T>(to_f32(x[c]) * inv_q * wq[c]);
  const long long slot = slot_mapping ? (long long)slot_mapping[t] : -1;
  if (slot < 0 || !k_pages) return;
  const int E = rank + rot;
  const long long page = slot / page_size;
  const int off = (int)(slot - page * page_size);
  T* kd = k_pages + (page * page_size + off) * (long long)E;
  T* vd = v_pages + page * (long long)E * page_size + off;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) {
    const T v = from_f32<T>(to_f32(x[kv_off + c]) * inv_k * wkv[c]);
    kd[c] = v;
    vd[(long long)c * page_size] = v;
  }
  const int half = rot_dims / 2;
  const T* kr = x + kv_off + rank;
  const float* cs = cos_sin + t * rot_dims;
  for (int c = threadIdx.x; c < rot; c += blockDim.x) {
    float v = to_f32(kr[c]);
    if (interleaved) {
      if (c < rot_dims) {
        const int i = c >> 1;
        v = (c & 1) ? v * cs[i] + to_f32(kr[c - 1]) * cs[half + i] : v * cs[i] - to_f32(kr[c + 1]) * cs[half + i];
      }
    } else if (c < half) v = v * cs[c] - to_f32(kr[c + half]) * cs[half + c];
    else if (c < rot_dims) v = v * cs[c - half] + to_f32(kr[c - half]) * cs[c];
    const T o = from_f32<T>(v);
    kd[rank + c] = o;
    vd[(long long)(rank + c) * page_size] = o;
  }
}

// ---------------------------------------------------------------- rotated query parts into the wide query
// q[t, h] = [ plain (dim) | to rotate (rot) ];  qe[t, h, rank : rank + rot] = rotate(q[t, h, dim:]).
// One block per token.
template <typename T>
__global__ void __launch_bounds__(256)
latent_query_rope_kernel(const T* __restrict__ q, long long ldq, T* __restrict__ qe, int heads, int dim, int rot,
                         int rot_dims, int rank, const float* __restrict__ cos_sin, int interleaved) {
  const long long t = blockIdx.x;
  const int half = rot_dims / 2;
  const float* cs = cos_sin + t * rot_dims;
  for (int i = threadIdx.x; i < heads * rot; i += blockDim.x) {
    const int h = i / rot, c = i - h * rot;
    const T* x = q + t * ldq + h * (long long)(dim + rot) + dim;
    float v = to_f32(x[c]);
    if (interleaved) {
      if (c < rot_dims) {
        const int i2 = c >> 1;
        v = (c & 1) ? v * cs[i2] + to_f32(x[c - 1]) * cs[half + i2] : v * cs[i2] - to_f32(x[c + 1]) * cs[half + i2];
      }
    } else if (c < half) v = v * cs[c] - to_f32(x[c + half]) * cs[half + c];
    else if (c < rot_dims) v = v * cs[c - half] + to_f32(x[c - half]) * cs[c];
    qe[(t * heads + h) * (long long)(rank + rot) + rank + c] = from_f32<T>(v);
  }
}

// ---------------------------------------------------------------- one small matrix per head
//   y[t, h * ys + n] = ( sum_k W[h][n][k] * x[t * ldx + h * xs + k] ) * ( g ? sigmoid(g[t * ldg + h * gn + (gn > 1 ? n : 0)]) : 1 )
// for n < N, k < K; gn = N: a gate per output element, gn = 1: one gate for all of a head's outputs.  Float accumulation in ascending k whatever the batch.  64 x 64 outputs a block of 256
// threads, k in slabs of 16 through LDS; blockIdx.z is the head.
#define HL_BM 64
#define HL_BN 64
#define HL_BK 16
template <typename T>
__global__ void __launch_bounds__(256)
head_linear_kernel(T* __restrict__ y, long long ldy, int ys, const T* __restrict__ x, long long ldx, int xs,
                   const T* __restrict__ W, int M, int N, int K, const T* __restrict__ g, long long ldg, int gn) {
  __shared__ float As[HL_BK][HL_BM + 4];
  __shared__ float Ws[HL_BK][HL_BN + 4];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * HL_BM, n0 = blockIdx.x * HL_BN;
  const T* Wh = W + (long long)h * N * K;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += HL_BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx >> 4, kk = idx & 15, k = k0 + kk;
      const int am = m0 + r, wn = n0 + r;
      As[kk][r] = (am < M && k < K) ? to_f32(x[(long long)am * ldx + (long long)h * xs + k]) : 0.f;
      Ws[kk][r] = (wn < N && k < K) ? to_f32(Wh[(long long)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HL_BK; ++kk) {
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
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (g) v *= 1.f / (1.f + expf(-to_f32(g[(long long)m * ldg + (long long)h * gn + (gn > 1 ? n : 0)])));
      y[(long long)m * ldy + (long long)h * ys + n] = from_f32<T>(v);
    }
  }
}

// The same for at most HL_ROWS rows (decode steps): a block takes 64 outputs of one head against all rows, the
// rows of x in LDS as floats; thread (n, part) sums its quarter of the inner size for every row, the quarters
// are added in their order.  Every W element is read once.
#define HL_ROWS 16
template <typename T>
__global__ void __launch_bounds__(256)
head_linear_rows_kernel(T* __restrict__ y, long long ldy, int ys, const T* __restrict__ x, long long ldx, int xs,
                        const T* __restrict__ W, int M, int N, int K, const T* __restrict__ g, long long ldg, int gn) {
  extern __shared__ float hl[];          // x [M][K] | partial sums [4][HL_ROWS][64]
  float* xr = hl;
  float* red = hl + M * K;
  const int h = blockIdx.y, n = blockIdx.x * 64 + (threadIdx.x & 63), part = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < M * K; i += 256) {
    const int t = i / K, k = i - t * K;
    xr[i] = to_f32(x[(long long)t * ldx + (long long)h * xs + k]);
  }
  __syncthreads();
  const int kq = (K + 3) / 4, k0 = part * kq, k1 = min(K, k0 + kq);
  const T* w = W + ((long long)h * N + min(n, N - 1)) * K;
  float acc[HL_ROWS];
#pragma unroll
  for (int t = 0; t < HL_ROWS; ++t) acc[t] = 0.f;
  // eight elements of the row of W are asked for before their products (a thread's time is its chain of loads)
  for (int kb = k0; kb < k1; kb += 8) {
    float wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) wv[u] = to_f32(w[min(kb + u, K - 1)]);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int k = kb + u;
      if (k < k1) {
#pragma unroll
        for (int t = 0; t < HL_ROWS; ++t)
          if (t < M) acc[t] = fmaf(xr[t * K + k], wv[u], acc[t]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < HL_ROWS; ++t) red[(part * HL_ROWS + t) * 64 + (threadIdx.x & 63)] = acc[t];
  __syncthreads();
  if (n >= N) return;
  for (int t = part; t < M; t += 4) {
    float v = 0.f;
#pragma unroll
    for (int p = 0; p < 4; ++p) v += red[(p * HL_ROWS + t) * 64 + (threadIdx.x & 63)];
    if (g) v *= 1.f / (1.f + expf(-to_f32(g[(long long)t * ldg + (long long)h * gn + (gn > 1 ? n : 0)])));
    y[(long long)t * ldy + (long long)h * ys + n] = from_f32<T>(v);
  }
}

// The same on the matrix cores (bfloat16; K, the head strides and the row strides multiples of 8): a wave takes
// 16 outputs of one head against 16 rows, both operands straight from global memory in 16-byte pieces
// (v_mfma_f32_16x16x32_bf16, A = 16 rows of W, B = 16 rows of x; the accumulator holds y^T[n = 4 lc + e][m = li]);
// the 4 waves of a block take 4 row tiles against the same 16 rows of W.  grid (N / 16, M / 64, heads).
typedef __bf16 hl_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hl_f32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(bf16_t* __restrict__ y, long long ldy, int ys, const bf16_t* __restrict__ x, long long ldx,
                        int xs, const bf16_t* __restrict__ W, int M, int N, int K, const bf16_t* __restrict__ g,
                        long long ldg, int gn) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 15, lc = lane >> 4;
  const int h = blockIdx.z, n0 = blockIdx.x * 16, m0 = (blockIdx.y * 4 + wave) * 16;
  if (m0 >= M) return;
  const bf16_t* wr = W + ((long long)h * N + min(n0 + li, N - 1)) * K;
  const bf16_t* xr = x + (long long)min(m0 + li, M - 1) * ldx + (long long)h * xs;
  const hl_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  hl_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 64) {        // two steps a turn: four loads asked for before the products
    const int ka = k0 + lc * 8, kb = ka + 32;
    const hl_bf16x8 a0 = *(const hl_bf16x8*)(wr + min(ka, K - 8)), b0 = *(const hl_bf16x8*)(xr + min(ka, K - 8));
    const hl_bf16x8 a1 = *(const hl_bf16x8*)(wr + min(kb, K - 8)), b1 = *(const hl_bf16x8*)(xr + min(kb, K - 8));
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, ka < K ? b0 : zero, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, kb < K ? b1 : zero, acc, 0, 0, 0);
  }
  const int m = m0 + li, nb = n0 + lc * 4;
  if (m >= M) return;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int n = nb + e;
    if (n >= N) continue;
    float v = acc[e];
    if (g) v *= 1.f / (1.f + expf(-(float)g[(long long)m * ldg + (long long)h * gn + (gn > 1 ? n : 0)]));
    y[(long long)m * ldy + (long long)h * ys + n] = (bf16_t)v;
  }
}

extern "C" int jv_head_linear_mfma_bf16(void* y, long long ldy, int ys, const void* x, long long ldx, int xs,
                                        const void* W, int M, int N, int K, int heads, const void* g, long long ldg,
                                        int gn, void* stream) {
  if (M <= 0 || N <= 0 || heads <= 0) return 0;
  if (g && gn != N && gn != 1) return (int)hipErrorInvalidValue;
  const unsigned gy = (M + 63) / 64;
  if (gy > 65535u || heads > 65535 || K < 8 || K % 8 || ldx % 8 || xs % 8) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(head_linear_mfma_kernel, dim3((N + 15) / 16, gy, heads), dim3(256), 0, (hipStream_t)stream,
                     (bf16_t*)y, ldy, ys, (const bf16_t*)x, ldx, xs, (const bf16_t*)W, M, N, K, (const bf16_t*)g, ldg, gn);
  return JV_LAUNCH_CHECK();
}

#define DEFINE_LATENT(SUF, T)                                                                              \
  extern "C" int jv_latent_prepare_##SUF(const void* proj, long long ld, int n, int q_rank, long long kv_off, \
                                         int rank,                                                         \
                                         int rot, int rot_dims, int interleaved, const float* wq,          \
                                         const float* wkv,                                                 \
                                         float eps, const float* cos_sin, const int* slot_mapping,         \
                                         void* cq, void* k_pages, void* v_pages, int page_size,            \
                                         void* stream) {                                                   \
    if (n <= 0) return 0;                                                                                  \
    if (q_rank < 0 || kv_off < 0 || rank <= 0 || rot < 0 || rot_dims < 0 || rot_dims > rot || rot_dims % 2 || \
        (q_rank && (!wq || !cq)))                                                                          \
      return (int)hipErrorInvalidValue;                                                                    \
    hipLaunchKernelGGL(latent_prepare_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t)stream,               \
                       (const T*)proj, ld, q_rank, kv_off, rank, rot, rot_dims, interleaved, wq, wkv, eps, cos_sin, \
                       slot_mapping, (T*)cq, (T*)k_pages, (T*)v_pages, page_size);                         \
    return JV_LAUNCH_CHECK();                                                                              \
  }                                                                                                        \
  extern "C" int jv_latent_query_rope_##SUF(const void* q, long long ldq, void* qe, int n, int heads, int dim, \
                                            int rot,                                                       \
                                            int rot_dims, int rank, const float* cos_sin, int interleaved, \
                                            void* stream) {                                                \
    if (n <= 0 || heads * rot <= 0) return 0;                                                              \
    if (rot_dims > rot || rot_dims % 2) return (int)hipErrorInvalidValue;                                  \
    hipLaunchKernelGGL(latent_query_rope_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t)stream,            \
                       (const T*)q, ldq, (T*)qe, heads, dim, rot, rot_dims, rank, cos_sin, interleaved);   \
    return JV_LAUNCH_CHECK();                                                                              \
  }                                                                                                        \
  extern "C" int jv_head_linear_##SUF(void* y, long long ldy, int ys, const void* x, long long ldx,        \
                                      int xs, const void* W, int M, int N, int K, int heads,               \
                                      const void* g, long long ldg, int gn, void* stream) {                \
    if (M <= 0 || N <= 0 || heads <= 0) return 0;                                                          \
    if (g && gn != N && gn != 1) return (int)hipErrorInvalidValue;                                         \
    const unsigned gy = (M + HL_BM - 1) / HL_BM;                                                           \
    if (gy > 65535u || heads > 65535 || K < 0) return (int)hipErrorInvalidValue;                           \
    if (M <= HL_ROWS && K > 0 && (size_t)(M * K + 4 * HL_ROWS * 64) * sizeof(float) <= 60 * 1024) {        \
      hipLaunchKernelGGL(head_linear_rows_kernel<T>, dim3((N + 63) / 64, heads), dim3(256),                \
                         (size_t)(M * K + 4 * HL_ROWS * 64) * sizeof(float), (hipStream_t)stream, (T*)y,   \
                         ldy, ys, (const T*)x, ldx, xs, (const T*)W, M, N, K, (const T*)g, ldg, gn);       \
      return JV_LAUNCH_CHECK();                                                                            \
    }                                                                                                      \
    hipLaunchKernelGGL(head_linear_kernel<T>, dim3((N + HL_BN - 1) / HL_BN, gy, heads), dim3(256), 0,      \
                       (hipStream_t)stream, (T*)y, ldy, ys, (const T*)x, ldx, xs, (const T*)W, M, N, K,    \
                       (const T*)g, ldg, gn);                                                              \
    return JV_LAUNCH_CHECK();                                                                              \
  }

DEFINE_LATENT(bf16, bf16_t)
DEFINE_LATENT(f32, float)
