// Norms of a layer arrangement that norms a sublayer's output before it joins the residual
// stream ("sandwich": x += N_b(f(N_a(x)))), and the gated norm behind a recurrent mixer.
// All sums, inverse roots and the residual stream are float.
#include "common.h"

// ---------------------------------------------------------------- post-norm + residual add + next pre-norm
// Row r = rows ? rows[i] : i.
//   v   = (y ? y[r] : 0) + parts[0][r] + parts[1][r] + ... (+ bias)   (the sublayer's output; parts added in order)
//   x   = h[r] + v * rsqrt(mean(v^2) + eps) * wb                 (float)
//         or, where wb is null (a sublayer's output that joins the stream under a constant only), h[r] + v * plain_scale
//   if (!rows) h[r] = x
//   if (out)   out[i] = T( x * rsqrt(mean(x^2) + eps_out) * w ),   or T(x) where w is null
// One block per output row; the row is kept in LDS between the passes (hidden floats).
template <typename T>
__global__ void __launch_bounds__(256)
postnorm_add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ y, const float* __restrict__ parts,
                            int n_parts, long long part_stride, const float* __restrict__ bias,
                            const float* __restrict__ wb,
                            const float* __restrict__ w, T* __restrict__ out, const int* __restrict__ rows,
                            int hidden, float eps, float eps_out, float plain_scale) {
  extern __shared__ float row[];
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float* hr = h + r * hidden;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = y ? to_f32(y[r * hidden + c]) : 0.f;
    for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + r * hidden + c];
    if (bias) v += bias[c];
    row[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv_b = wb ? rsqrtf(ss / (float)hidden + eps) : plain_scale;
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float x = hr[c] + row[c] * inv_b * (wb ? wb[c] : 1.f);
    if (!rows) hr[c] = x;
    row[c] = x;
    ss2 += x * x;
  }
  if (!out) return;
  T* o = out + i * hidden;
  if (!w) {          // the reader takes the stream itself: no norm, the row in the activation type
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) o[c] = from_f32<T>(row[c]);
    return;
  }
  ss2 = block_sum(ss2, red);
  const float inv = rsqrtf(ss2 / (float)hidden + eps_out);
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) o[c] = from_f32<T>(row[c] * inv * w[c]);
}

// ---------------------------------------------------------------- norm of float rows times a sigmoid gate
//   out[t, c] = T( o[t, c] * rsqrt(mean_c(o[t]^2) + eps) * w[c] * sigmoid(g[t * g_stride + c]) )
// o is float (the output of a recurrence), g lives in a wider row of the activation type.
template <typename T>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g,
                     long long g_stride, const float* __restrict__ w, int width, float eps) {
  __shared__ float red[32];
  const long long t = blockIdx.x;
  const float* x = o + t * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) ss += x[c] * x[c];
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float gate = 1.f / (1.f + expf(-to_f32(g[t * g_stride + c])));
    out[t * width + c] = from_f32<T>(x[c] * inv * w[c] * gate);
  }
}

// The same for widths that are multiples of 4: 16 bytes of the float arrays a lane, every load of a pass asked
// for before the sums (a decode step has few rows: what a row costs is its chain of dependent loads).
template <typename T> struct SnVec4;
template <> struct SnVec4<float> { typedef float4 type; };
template <> struct SnVec4<bf16_t> { typedef __attribute__((ext_vector_type(4))) __bf16 type; };
template <typename T> __device__ __forceinline__ float4 sn_load4(const T* p) {
  const typename SnVec4<T>::type v = *(const typename SnVec4<T>::type*)p;
  return float4{to_f32<T>(v[0]), to_f32<T>(v[1]), to_f32<T>(v[2]), to_f32<T>(v[3])};
}
template <> __device__ __forceinline__ float4 sn_load4<float>(const float* p) { return *(const float4*)p; }
template <typename T> __device__ __forceinline__ void sn_store4(T* p, float4 v) {
  typename SnVec4<T>::type o;
  o[0] = from_f32<T>(v.x); o[1] = from_f32<T>(v.y); o[2] = from_f32<T>(v.z); o[3] = from_f32<T>(v.w);
  *(typename SnVec4<T>::type*)p = o;
}
template <> __device__ __forceinline__ void sn_store4<float>(float* p, float4 v) { *(float4*)p = v; }

#define SN_V 4      // 16-byte pieces a thread: rows of up to 4 * SN_V * 256 = 4,096 floats
template <typename T>
__global__ void __launch_bounds__(256)
postnorm_add_rmsnorm_vec_kernel(float* __restrict__ h, const T* __restrict__ y, const float* __restrict__ parts,
                                int n_parts, long long part_stride, const float* __restrict__ bias,
                                const float* __restrict__ wb,
                                const float* __restrict__ w, T* __restrict__ out, const int* __restrict__ rows,
                                int hidden, float eps, float eps_out, float plain_scale) {
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float4 v[SN_V], x[SN_V], b[SN_V];
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < SN_V; ++q) {
    const int c = (threadIdx.x + q * 256) * 4;
    const int cc = c < hidden ? c : 0;           // a piece beyond the row reads the row's first piece, its share is left out
    v[q] = y ? sn_load4<T>(y + r * hidden + cc) : float4{0.f, 0.f, 0.f, 0.f};
    x[q] = *(const float4*)(h + r * hidden + cc);
    b[q] = wb ? *(const float4*)(wb + cc) : float4{1.f, 1.f, 1.f, 1.f};
  }
  for (int p = 0; p < n_parts; ++p) {
#pragma unroll
    for (int q = 0; q < SN_V; ++q) {
      const int c = (threadIdx.x + q * 256) * 4;
      const float4 t = *(const float4*)(parts + p * part_stride + r * hidden + (c < hidden ? c : 0));
      v[q].x += t.x; v[q].y += t.y; v[q].z += t.z; v[q].w += t.w;
    }
  }
  if (bias) {
#pragma unroll
    for (int q = 0; q < SN_V; ++q) {
      const int c = (threadIdx.x + q * 256) * 4;
      const float4 t = *(const float4*)(bias + (c < hidden ? c : 0));
      v[q].x += t.x; v[q].y += t.y; v[q].z += t.z; v[q].w += t.w;
    }
  }
#pragma unroll
  for (int q = 0; q < SN_V; ++q)
    if ((threadIdx.x + q * 256) * 4 < hidden) ss += v[q].x * v[q].x + v[q].y * v[q].y + v[q].z * v[q].z + v[q].w * v[q].w;
  ss = block_sum(ss, red);
  const float inv_b = wb ? rsqrtf(ss / (float)hidden + eps) : plain_scale;
  float ss2 = 0.f;
#pragma unroll
  for (int q = 0; q < SN_V; ++q) {
    const int c = (threadIdx.x + q * 256) * 4;
    x[q].x += v[q].x * inv_b * b[q].x; x[q].y += v[q].y * inv_b * b[q].y;
    x[q].z += v[q].z * inv_b * b[q].z; x[q].w += v[q].w * inv_b * b[q].w;
    if (c < hidden) {
      if (!rows) *(float4*)(h + r * hidden + c) = x[q];
      ss2 += x[q].x * x[q].x + x[q].y * x[q].y + x[q].z * x[q].z + x[q].w * x[q].w;
    }
  }
  if (!out) return;
  if (!w) {          // the reader takes the stream itself: no norm, the row in the activation type
#pragma unroll
    for (int q = 0; q < SN_V; ++q) {
      const int c = (threadIdx.x + q * 256) * 4;
      if (c < hidden) sn_store4<T>(out + i * hidden + c, x[q]);
    }
    return;
  }
  ss2 = block_sum(ss2, red);
  const float inv = rsqrtf(ss2 / (float)hidden + eps_out);
#pragma unroll
  for (int q = 0; q < SN_V; ++q) {
    const int c = (threadIdx.x + q * 256) * 4;
    if (c < hidden) {
      const float4 g = *(const float4*)(w + c);
      sn_store4<T>(out + i * hidden + c, float4{x[q].x * inv * g.x, x[q].y * inv * g.y, x[q].z * inv * g.z, x[q].w * inv * g.w});
    }
  }
}

#define DEFINE_SANDWICH(SUF, T)                                                                          \
  extern "C" int jv_postnorm_add_rmsnorm_##SUF(float* h, const void* y, const float* parts, int n_parts, \
                                               long long part_stride, const float* bias,               \
                                               const float* wb, const float* w,                         \
                                               void* out, const int* rows, int n_out, int hidden,        \
                                               float eps, float eps_out, float plain_scale,              \
                                               void* stream) {                                           \
    if (n_out <= 0 || hidden <= 0) return 0;                                                             \
    if ((!y && n_parts <= 0) || hidden > 16384) return (int)hipErrorInvalidValue;                        \
    if (hidden % 4 == 0 && hidden <= 4 * SN_V * 256) {                                                   \
      hipLaunchKernelGGL(postnorm_add_rmsnorm_vec_kernel<T>, dim3(n_out), dim3(256), 0,                  \
                         (hipStream_t)stream, h, (const T*)y, parts, n_parts, part_stride, bias, wb, w,  \
                         (T*)out, rows, hidden, eps, eps_out, plain_scale);                              \
      return JV_LAUNCH_CHECK();                                                                          \
    }                                                                                                    \
    hipLaunchKernelGGL(postnorm_add_rmsnorm_kernel<T>, dim3(n_out), dim3(256), hidden * sizeof(float),   \
                       (hipStream_t)stream, h, (const T*)y, parts, n_parts, part_stride, bias, wb, w,    \
                       (T*)out,                                                                          \
                       rows, hidden, eps, eps_out, plain_scale);                                         \
    return JV_LAUNCH_CHECK();                                                                            \
  }                                                                                                      \
  extern "C" int jv_gated_rmsnorm_##SUF(void* out, const float* o, const void* g, long long g_stride,    \
                                        const float* w, int n, int width, float eps, void* stream) {     \
    if (n <= 0 || width <= 0) return 0;                                                                  \
    hipLaunchKernelGGL(gated_rmsnorm_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t)stream, (T*)out, o,  \
                       (const T*)g, g_stride, w, width, eps);                                            \
    return JV_LAUNCH_CHECK();                                                                            \
  }

DEFINE_SANDWICH(bf16, bf16_t)
DEFINE_SANDWICH(f32, float)
