// Small kernels of a layer whose mixer and feed-forward read ONE normed input and join the stream together,
// of an embedding that adds a row chosen by the pair (previous token, token), of a per-layer input that is
// looked up by the token itself, of a sigmoid gate on attention heads, and the soft cap on logits.
// The residual stream and every sum are float.
#include "common.h"

// ---------------------------------------------------------------- embedding + row of a hashed token pair
// h[t] = float(table[ids[t]]) + float(pair[r]),  r = prev[t] < 0 ? spare : (prev[t] * mul_prev + ids[t] * mul_cur) mod buckets
// (64-bit integers; `spare` is the table's last row, taken by a sequence's first token).  An id outside
// [0, rows) makes its row NaN, as in the plain gather.  One block per token.
template <typename T>
__global__ void __launch_bounds__(256)
embedding_pair_kernel(float* __restrict__ h, const T* __restrict__ table, const T* __restrict__ pair,
                      const int* __restrict__ ids, const int* __restrict__ prev, int hidden, int rows,
                      long long buckets, long long mul_prev, long long mul_cur, float scale) {
  const long long t = blockIdx.x;
  const int id = ids[t], pv = prev[t];
  const bool inside = id >= 0 && id < rows && pv < rows;
  const long long r = pv < 0 ? buckets : (((long long)pv * mul_prev + (long long)id * mul_cur) % buckets);
  const T* a = table + (long long)(inside ? id : 0) * hidden;
  const T* b = pair ? pair + (inside ? r : 0) * hidden : nullptr;     // no second table: the scaled row alone
  float* out = h + t * hidden;
  const float nan = __builtin_nanf("");
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float v = to_f32(a[c]) * scale + (b ? to_f32(b[c]) : 0.f);
    out[c] = inside ? v : nan;
  }
}

// ---------------------------------------------------------------- two sublayers' outputs join the stream
//   s = (ya + pa[0] + pa[1] + ...) + (yb + pb[0] + ...);   h += s;   out = T(h)  (if out)
// ya, yb rows of the activation type or null; pa, pb float stacks of partial results or null.
// V = 4: every pointer and stride allows 16-byte pieces of the float arrays (8 bytes of bfloat16).
template <typename T, int V> struct PlVec { typedef T type __attribute__((ext_vector_type(V))); };
template <typename T> struct PlVec<T, 1> { typedef T type; };
template <typename T, int V>
__device__ __forceinline__ void pl_load(const T* p, float (&v)[V]) {
  if constexpr (V == 1) {
    v[0] = to_f32(*p);
  } else {
    const typename PlVec<T, V>::type x = *(const typename PlVec<T, V>::type*)p;
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = to_f32<T>(x[e]);
  }
}
template <typename T, int V>
__device__ __forceinline__ void pl_store(T* p, const float (&v)[V]) {
  if constexpr (V == 1) {
    *p = from_f32<T>(v[0]);
  } else {
    typename PlVec<T, V>::type x;
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = from_f32<T>(v[e]);
    *(typename PlVec<T, V>::type*)p = x;
  }
}

template <typename T, int V>
__global__ void __launch_bounds__(256)
add_outputs_kernel(float* __restrict__ h, const T* __restrict__ ya, const float* __restrict__ pa, int na,
                   long long sa, const T* __restrict__ yb, const float* __restrict__ pb, int nb, long long sb,
                   T* __restrict__ out, long long n) {
  const long long i0 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (i0 >= n) return;
  float a[V], b[V], x[V], t[V];
#pragma unroll
  for (int e = 0; e < V; ++e) a[e] = b[e] = 0.f;
  pl_load<float, V>(h + i0, x);
  if (ya) pl_load<T, V>(ya + i0, a);
  if (yb) pl_load<T, V>(yb + i0, b);
  for (int p = 0; p < na; ++p) {
    pl_load<float, V>(pa + p * sa + i0, t);
#pragma unroll
    for (int e = 0; e < V; ++e) a[e] += t[e];
  }
  for (int p = 0; p < nb; ++p) {
    pl_load<float, V>(pb + p * sb + i0, t);
#pragma unroll
    for (int e = 0; e < V; ++e) b[e] += t[e];
  }
#pragma unroll
  for (int e = 0; e < V; ++e) x[e] += a[e] + b[e];
  pl_store<float, V>(h + i0, x);
  if (out) pl_store<T, V>(out + i0, x);
}

// ---------------------------------------------------------------- gate of a per-layer token input
// z[t, c] = act(z[t, c]) * float(table[ids[t], offset + c]),  c < dim, in place; table rows are `width` wide.
template <typename T>
__global__ void __launch_bounds__(256)
token_gate_mul_kernel(T* __restrict__ z, const T* __restrict__ table, const int* __restrict__ ids, long long n,
                      int dim, int width, int offset, int rows, int act) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * dim) return;
  const long long t = i / dim;
  const int c = (int)(i - t * dim);
  const int id = ids[t];
  const bool inside = id >= 0 && id < rows;
  const float e = inside ? to_f32(table[(long long)id * width + offset + c]) : __builtin_nanf("");
  z[i] = from_f32<T>(jv_act(act, to_f32(z[i])) * e);
}

// ---------------------------------------------------------------- sigmoid gate on attention heads
// o[t, h * dp + i] *= sigmoid(g[t * ldg + h * dv + i]),  i < dv  (heads of o padded to dp >= dv), in place.
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_gate_heads_kernel(T* __restrict__ o, const T* __restrict__ g, long long ldg, long long n, int heads, int dv,
                          int dp) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long per = (long long)heads * dv;
  if (i >= n * per) return;
  const long long t = i / per;
  const int r = (int)(i - t * per);
  const int hd = r / dv, e = r - hd * dv;
  T* p = o + (t * heads + hd) * dp + e;
  const float gate = 1.f / (1.f + expf(-to_f32(g[t * ldg + r])));
  *p = from_f32<T>(to_f32(*p) * gate);
}

// The same with 16 bytes a lane, where the head sizes, the gate's row stride and both addresses allow it.
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_gate_heads_vec_kernel(T* __restrict__ o, const T* __restrict__ g, long long ldg, long long n, int heads, int dv,
                              int dp) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T tv __attribute__((ext_vector_type(V)));
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long per = (long long)heads * dv / V;
  if (i >= n * per) return;
  const long long t = i / per;
  const int r = (int)(i - t * per) * V;
  const int hd = r / dv, e = r - hd * dv;
  tv* p = (tv*)(o + (t * heads + hd) * dp + e);
  const tv gv = *(const tv*)(g + t * ldg + r);
  tv ov = *p;
#pragma unroll
  for (int k = 0; k < V; ++k) ov[k] = from_f32<T>(to_f32(ov[k]) / (1.f + expf(-to_f32(gv[k]))));
  *p = ov;
}

// ---------------------------------------------------------------- soft cap on float logits
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ x, long long n, float cap) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int jv_softcap_f32(float* x, long long n, float cap, void* stream) {
  if (n <= 0) return 0;
  if (!(cap > 0.f) || (n + 255) / 256 > 0x7fffffffll) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, n, cap);
  return JV_LAUNCH_CHECK();
}

template <typename T, int V>
static int launch_add_outputs(float* h, const void* ya, const float* pa, int na, long long sa, const void* yb,
                              const float* pb, int nb, long long sb, void* out, long long n, void* stream) {
  const long long threads = (n + V - 1) / V;
  if ((threads + 255) / 256 > 0x7fffffffll) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL((add_outputs_kernel<T, V>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, h, (const T*)ya, pa, na, sa, (const T*)yb, pb, nb, sb, (T*)out, n);
  return JV_LAUNCH_CHECK();
}

#define DEFINE_PARALLEL_LAYER(SUF, T)                                                                             \
  extern "C" int jv_embedding_pair_##SUF(float* h, const void* table, const void* pair, const int* ids,           \
                                         const int* prev, int n_tokens, int hidden, int rows, long long buckets,  \
                                         long long mul_prev, long long mul_cur, float scale, void* stream) {      \
    if (n_tokens <= 0) return 0;                                                                                  \
    if (buckets <= 0 || mul_prev < 0 || mul_cur < 0 || mul_prev > 0x7fffffffll || mul_cur > 0x7fffffffll)         \
      return (int)hipErrorInvalidValue;                                                                           \
    hipLaunchKernelGGL(embedding_pair_kernel<T>, dim3(n_tokens), dim3(256), 0, (hipStream_t)stream, h,            \
                       (const T*)table, (const T*)pair, ids, prev, hidden, rows, buckets, mul_prev, mul_cur, scale); \
    return JV_LAUNCH_CHECK();                                                                                     \
  }                                                                                                               \
  /* n = rows * hidden elements; the stacks' strides in elements; `vec`: every pointer and stride allows 4 */    \
  extern "C" int jv_add_outputs_##SUF(float* h, const void* ya, const float* pa, int na, long long sa,            \
                                      const void* yb, const float* pb, int nb, long long sb, void* out,           \
                                      long long n, int vec, void* stream) {                                       \
    if (n <= 0) return 0;                                                                                         \
    if (na < 0 || nb < 0 || (na && !pa) || (nb && !pb)) return (int)hipErrorInvalidValue;                         \
    return vec ? launch_add_outputs<T, 4>(h, ya, pa, na, sa, yb, pb, nb, sb, out, n, stream)                      \
               : launch_add_outputs<T, 1>(h, ya, pa, na, sa, yb, pb, nb, sb, out, n, stream);                     \
  }                                                                                                               \
  extern "C" int jv_token_gate_mul_##SUF(void* z, const void* table, const int* ids, long long n, int dim,        \
                                         int width, int offset, int rows, int act, void* stream) {                \
    if (n <= 0 || dim <= 0) return 0;                                                                             \
    if (offset < 0 || offset + dim > width || (act && !jv_plain_act_known(act)) ||                                \
        (n * dim + 255) / 256 > 0x7fffffffll)                                                                     \
      return (int)hipErrorInvalidValue;                                                                           \
    hipLaunchKernelGGL(token_gate_mul_kernel<T>, dim3((unsigned)((n * dim + 255) / 256)), dim3(256), 0,           \
                       (hipStream_t)stream, (T*)z, (const T*)table, ids, n, dim, width, offset, rows, act);       \
    return JV_LAUNCH_CHECK();                                                                                     \
  }                                                                                                               \
  extern "C" int jv_sigmoid_gate_heads_##SUF(void* o, const void* g, long long ldg, long long n, int heads,       \
                                             int dv, int dp, void* stream) {                                      \
    if (n <= 0 || heads <= 0 || dv <= 0) return 0;                                                                \
    if (dp < dv || ldg < (long long)heads * dv || (n * heads * dv + 255) / 256 > 0x7fffffffll)                    \
      return (int)hipErrorInvalidValue;                                                                           \
    constexpr int V = 16 / (int)sizeof(T);                                                                        \
    if (dv % V == 0 && dp % V == 0 && ldg % V == 0 && (uintptr_t)o % 16 == 0 && (uintptr_t)g % 16 == 0) {         \
      const long long items = n * heads * dv / V;                                                                 \
      hipLaunchKernelGGL(sigmoid_gate_heads_vec_kernel<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,   \
                         (hipStream_t)stream, (T*)o, (const T*)g, ldg, n, heads, dv, dp);                         \
      return JV_LAUNCH_CHECK();                                                                                   \
    }                                                                                                             \
    hipLaunchKernelGGL(sigmoid_gate_heads_kernel<T>, dim3((unsigned)((n * heads * dv + 255) / 256)), dim3(256),   \
                       0, (hipStream_t)stream, (T*)o, (const T*)g, ldg, n, heads, dv, dp);                        \
    return JV_LAUNCH_CHECK();                                                                                     \
  }

DEFINE_PARALLEL_LAYER(bf16, bf16_t)
DEFINE_PARALLEL_LAYER(f32, float)
