// Time mixing with a decay per key channel and a bonus for the current token, and what stands before it:
//
//   token_shift_mix   several blends of every row with the row before it in its request,
//                       out[s][t] = x[t] + (x[t-1] - x[t]) * mu[s]
//                     where the row before a request's first row of the step is the request's state row (zeros for a
//                     request that starts); the state then takes the request's last row of the step
//   wkv_steps         per head, S [dim][vdim] the request's float state:
//                       w_t = exp(-exp(rate_t + w0))                       (per key channel, float)
//                       o_t = S^T r_t + (sum_d r_t[d] u[d] k_t[d]) v_t     (the bonus u counts for the current token only)
//                       S   <- diag(w_t) S + k_t v_t^T
//   wkv_chunks        the same by chunks of WKV_LC tokens, for prompt portions (see below)
//
// r, k, v and the decay's rate are products in the activation type; everything from there on is float.  The state of a
// request lives in a row of `state` [slots + 1][heads][dim][vdim] between steps.  Columns of S never mix, so a block
// takes one (request, head, slice of columns) and a thread keeps up to WKV_ROWS rows of one column in registers.
#include "common.h"

#define WKV_ROWS 32

// ---------------------------------------------------------------- blends with the previous row
// grid (tokens, column blocks of 256); mu [n_mix][hidden] float; out [n_mix][n][hidden]; state [slots + 1][hidden] float.
// Only the block of a request's first row of the step reads the state, and it writes it too, column by column after
// its read: the row that the step leaves is x[last row of the request].
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_mix_kernel(T* __restrict__ out, const T* __restrict__ x, const float* __restrict__ mu, int n_mix,
                       float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_seqlens,
                       const int* __restrict__ token_req, long long n, int hidden) {
  const long long t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= hidden) return;
  const int r = token_req[t];
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  const float cur = to_f32(x[t * hidden + c]);
  float before;
  if (t > t0) {
    before = to_f32(x[(t - 1) * hidden + c]);
  } else {
    float* st = state + (long long)slot_ids[r] * hidden + c;
    before = *st;
    *st = to_f32(x[(long long)(t1 - 1) * hidden + c]);
  }
  const float d = before - cur;
  for (int s = 0; s < n_mix; ++s)
    out[((long long)s * n + t) * hidden + c] = from_f32<T>(fmaf(d, mu[(long long)s * hidden + c], cur));
}

// ---------------------------------------------------------------- the recurrence, token by token
// grid (requests, heads, column slices); block 256 = parts x cols threads, cols a power of two.
// r, k, rate: [n][heads][dim] with row strides ldr, ldk, ldw; v [n][heads][vdim] with row stride ldv; w0, u [heads][dim]
// float; out [n][heads * vdim] float.
template <typename T>
__global__ void __launch_bounds__(256)
wkv_steps_kernel(float* __restrict__ out, const T* __restrict__ rr, long long ldr, const T* __restrict__ kk,
                 long long ldk, const T* __restrict__ vv, long long ldv, const T* __restrict__ rate, long long ldw,
                 const float* __restrict__ w0, const float* __restrict__ bonus, float* __restrict__ state,
                 const int* __restrict__ slot_ids, const int* __restrict__ cu_seqlens, int heads, int dim, int vdim,
                 int cols) {
  extern __shared__ float lds[];          // 2 x (r[dim] | k[dim] | w[dim] | v[cols]) | partial sums [parts][cols]
  const int q = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * cols;
  const int parts = blockDim.x / cols;
  const int col = threadIdx.x % cols, part = threadIdx.x / cols;
  const int t0 = cu_seqlens[q], t1 = cu_seqlens[q + 1];
  if (t1 <= t0) return;
  const int stage = 3 * dim + cols;
  float* red = lds + 2 * stage;
  const bool live = c0 + col < vdim;
  float* S = state + (((long long)slot_ids[q] * heads + h) * dim) * vdim + c0 + col;
  float s[WKV_ROWS], ub[WKV_ROWS];
#pragma unroll
  for (int i = 0; i < WKV_ROWS; ++i) {
    const int d = part + i * parts;
    s[i] = (live && d < dim) ? S[(long long)d * vdim] : 0.f;
    ub[i] = d < dim ? bonus[h * dim + d] : 0.f;
  }
  for (int t = t0; t < t1; ++t) {
    float* buf = lds + ((t - t0) & 1) * stage;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
      buf[d] = to_f32(rr[(long long)t * ldr + h * dim + d]);
      buf[dim + d] = to_f32(kk[(long long)t * ldk + h * dim + d]);
      buf[2 * dim + d] = expf(-expf(to_f32(rate[(long long)t * ldw + h * dim + d]) + w0[h * dim + d]));
    }
    if (threadIdx.x < cols)
      buf[3 * dim + threadIdx.x] = (c0 + threadIdx.x < vdim) ? to_f32(vv[(long long)t * ldv + h * vdim + c0 + threadIdx.x]) : 0.f;
    __syncthreads();
    const float v = buf[3 * dim + col];
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < WKV_ROWS; ++i) {
      const int d = part + i * parts;
      if (d < dim) {
        const float kv = buf[dim + d] * v;
        acc = fmaf(buf[d], fmaf(ub[i], kv, s[i]), acc);
        s[i] = fmaf(buf[2 * dim + d], s[i], kv);
      }
    }
    red[part * cols + col] = acc;
    __syncthreads();
    if (part == 0 && live) {
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += red[p * cols + col];
      out[(long long)t * heads * vdim + h * vdim + c0 + col] = o;
    }
    // the next token fills the other stage; red is rewritten only behind the barrier after that fill
  }
#pragma unroll
  for (int i = 0; i < WKV_ROWS; ++i) {
    const int d = part + i * parts;
    if (live && d < dim) S[(long long)d * vdim] = s[i];
  }
}

extern "C" int jv_wkv_max_dim() { return WKV_ROWS * 256; }

#define DEFINE_WKV(SUF, T)                                                                                      \
  extern "C" int jv_token_shift_mix_##SUF(void* out, const void* x, const float* mu, int n_mix, float* state,   \
                                          const int* slot_ids, const int* cu_seqlens, const int* token_req,     \
                                          long long n, int hidden, void* stream) {                              \
    if (n <= 0 || hidden <= 0 || n_mix <= 0) return 0;                                                          \
    if (n > 0x7fffffffll || (hidden + 255) / 256 > 65535) return (int)hipErrorInvalidValue;                     \
    hipLaunchKernelGGL(token_shift_mix_kernel<T>, dim3((unsigned)n, (hidden + 255) / 256), dim3(256), 0,        \
                       (hipStream_t)stream, (T*)out, (const T*)x, mu, n_mix, state, slot_ids, cu_seqlens,       \
                       token_req, n, hidden);                                                                   \
    return JV_LAUNCH_CHECK();                                                                                   \
  }                                                                                                             \
  extern "C" int jv_wkv_steps_##SUF(float* out, const void* r, long long ldr, const void* k, long long ldk,     \
                                    const void* v, long long ldv, const void* rate, long long ldw,              \
                                    const float* w0, const float* bonus, float* state, const int* slot_ids,     \
                                    const int* cu_seqlens, int n_requests, int heads, int dim, int vdim,        \
                                    void* stream) {                                                             \
    if (n_requests <= 0 || heads <= 0) return 0;                                                                \
    if (dim <= 0 || vdim <= 0 || heads > 65535) return (int)hipErrorInvalidValue;                               \
    int cols = 64;                       /* the widest slice that keeps a thread's rows in registers */         \
    while (cols > 1 && (cols / 2 >= vdim || (long long)dim * cols > 256LL * WKV_ROWS)) cols /= 2;               \
    if ((long long)dim * cols > 256LL * WKV_ROWS) return (int)hipErrorInvalidValue;                             \
    const int parts = 256 / cols;                                                                               \
    const size_t shmem = (2 * (3 * dim + cols) + parts * cols) * sizeof(float);                                 \
    if (shmem > 64 * 1024 || (vdim + cols - 1) / cols > 65535) return (int)hipErrorInvalidValue;                \
    hipLaunchKernelGGL(wkv_steps_kernel<T>, dim3(n_requests, heads, (vdim + cols - 1) / cols), dim3(256),       \
                       shmem, (hipStream_t)stream, out, (const T*)r, ldr, (const T*)k, ldk, (const T*)v, ldv,   \
                       (const T*)rate, ldw, w0, bonus, state, slot_ids, cu_seqlens, heads, dim, vdim, cols);    \
    return JV_LAUNCH_CHECK();                                                                                   \
  }

DEFINE_WKV(bf16, bf16_t)
DEFINE_WKV(f32, float)
