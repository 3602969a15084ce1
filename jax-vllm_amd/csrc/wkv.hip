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
//   wkv_chunks        the same by chunks of 32 tokens, for prompt portions (see below)
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

// The same with 16 bytes a lane, where the width and the addresses allow it.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_mix_vec_kernel(T* __restrict__ out, const T* __restrict__ x, const float* __restrict__ mu, int n_mix,
                           float* __restrict__ state, const int* __restrict__ slot_ids,
                           const int* __restrict__ cu_seqlens, const int* __restrict__ token_req, long long n,
                           int hidden) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T tv __attribute__((ext_vector_type(V)));
  const long long t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= hidden) return;
  const int r = token_req[t];
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  const tv cv = *(const tv*)(x + t * hidden + c);
  float cur[V], d[V];
  if (t > t0) {
    const tv bv = *(const tv*)(x + (t - 1) * hidden + c);
#pragma unroll
    for (int e = 0; e < V; ++e) { cur[e] = to_f32(cv[e]); d[e] = to_f32(bv[e]) - cur[e]; }
  } else {
    float* st = state + (long long)slot_ids[r] * hidden + c;
    const tv lv = *(const tv*)(x + (long long)(t1 - 1) * hidden + c);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      cur[e] = to_f32(cv[e]);
      d[e] = st[e] - cur[e];
      st[e] = to_f32(lv[e]);
    }
  }
  for (int s = 0; s < n_mix; ++s) {
    tv ov;
#pragma unroll
    for (int e = 0; e < V; ++e) ov[e] = from_f32<T>(fmaf(d[e], mu[(long long)s * hidden + c + e], cur[e]));
    *(tv*)(out + ((long long)s * n + t) * hidden + c) = ov;
  }
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

// ---------------------------------------------------------------- the recurrence by chunks
// With l_t = max(log w_t, -WKV_MIN_LOG) per key channel (a decay below e^-64 is nothing in float), b_t = l_0 + ... + l_t
// inside a chunk of n <= WKV_LC tokens (b_-1 = 0) and S0 the state before the chunk:
//     o_t   = (r_t * exp(b_(t-1)))^T S0 + sum_{j<t} a[t][j] v_j + a[t][t] v_t
//     a[t][j] = sum_c r_t[c] k_j[c] exp(b_(t-1)[c] - b_j[c])  (j < t),     a[t][t] = sum_c r_t[c] u[c] k_t[c]
//     S_end = diag(exp(b_(n-1))) S0 + sum_j (k_j * exp(b_(n-1) - b_j)) v_j^T
// Only differences <= 0 are exponentiated, channel by channel (no product of a grown query with a shrunk key, which
// would overflow).  Three launches, so that the chunks of a long prompt run side by side and only the cheap part is serial:
//   local:  per (chunk, head)   out_t = sum_j a[t][j] v_j;  U = sum_j k'_j v_j^T -> scratch[chunk];  r_t * exp(b_(t-1)) -> rq;
//                               exp(b_(n-1)) -> dtot[chunk]
//   scan:   per (request, head) for its chunks in order: scratch[chunk] <- S (the state BEFORE the chunk),
//                               S <- diag(dtot[chunk]) S + U;  at the end state <- S
//   apply:  per (chunk, head)   out_t += rq_t^T S_before
#define WKV_LC 32
#define WKV_CW 64          // columns of v a block takes at a time
#define WKV_MIN_LOG 64.f

// e^x for x in [-32 * WKV_MIN_LOG, 0] through the hardware's 2^x: the argument's rounding costs |x| e^x 2^-24 at most,
// below a hundred-millionth absolutely, which is the float rounding of the sums these weights enter.
__device__ __forceinline__ float wkv_exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

template <typename T>
__global__ void __launch_bounds__(256)
wkv_local_kernel(float* __restrict__ out, float* __restrict__ scratch, float* __restrict__ rq, float* __restrict__ dtot,
                 const T* __restrict__ rr, long long ldr, const T* __restrict__ kk, long long ldk,
                 const T* __restrict__ vv, long long ldv, const T* __restrict__ rate, long long ldw,
                 const float* __restrict__ w0, const float* __restrict__ bonus, const int* __restrict__ work,
                 const int* __restrict__ cu_seqlens, int heads, int dim, int vdim) {
  extern __shared__ float lds[];      // r [LC][dim + 1] | k [LC][dim + 1] | b [LC][dim + 1] | a [LC][LC + 1] | v [LC][CW] | u [dim]
  const int ld = dim + 1;
  float* rs = lds;
  float* ks = rs + WKV_LC * ld;
  float* bs = ks + WKV_LC * ld;
  float* as = bs + WKV_LC * ld;
  float* vs = as + WKV_LC * (WKV_LC + 1);
  float* us = vs + WKV_LC * WKV_CW;
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  for (int c = tid; c < dim; c += 256) us[c] = bonus[h * dim + c];
  const int req = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(WKV_LC, cu_seqlens[req + 1] - b0);
  for (int i = tid; i < WKV_LC * dim; i += 256) {
    const int t = i / dim, c = i - t * dim;
    float r = 0.f, k = 0.f, l = 0.f;
    if (t < n) {
      const long long row = b0 + t;
      r = to_f32(rr[row * ldr + h * dim + c]);
      k = to_f32(kk[row * ldk + h * dim + c]);
      l = fmaxf(-expf(to_f32(rate[row * ldw + h * dim + c]) + w0[h * dim + c]), -WKV_MIN_LOG);
    }
    rs[t * ld + c] = r;
    ks[t * ld + c] = k;
    bs[t * ld + c] = l;
  }
  __syncthreads();
  for (int c = tid; c < dim; c += 256) {
    float run = 0.f;
    for (int t = 0; t < WKV_LC; ++t) {
      const float before = run;
      run += bs[t * ld + c];
      bs[t * ld + c] = run;
      if (t < n) rq[(long long)(b0 + t) * heads * dim + h * dim + c] = rs[t * ld + c] * wkv_exp_neg(before);
    }
    dtot[((long long)ch * heads + h) * dim + c] = wkv_exp_neg(run);
  }
  __syncthreads();
  for (int e = tid; e < WKV_LC * WKV_LC; e += 256) {
    const int t = e / WKV_LC, j = e - t * WKV_LC;
    float a = 0.f;
    if (j < t) {
#pragma unroll 4
      for (int c = 0; c < dim; ++c)
        a = fmaf(rs[t * ld + c] * ks[j * ld + c], wkv_exp_neg(bs[(t - 1) * ld + c] - bs[j * ld + c]), a);
    } else if (j == t) {
      for (int c = 0; c < dim; ++c) a = fmaf(rs[t * ld + c] * ks[t * ld + c], us[c], a);
    }
    as[t * (WKV_LC + 1) + j] = a;
  }
  __syncthreads();
  for (int i = tid; i < WKV_LC * dim; i += 256) {
    const int t = i / dim, c = i - t * dim;
    ks[t * ld + c] *= wkv_exp_neg(bs[(WKV_LC - 1) * ld + c] - bs[t * ld + c]);
  }
  const int col = tid & (WKV_CW - 1), tq = tid / WKV_CW;      // tq is the same for all lanes of a wave
  for (int c0 = 0; c0 < vdim; c0 += WKV_CW) {
    __syncthreads();      // k' is complete (first turn); the last turn's readers of v are done
    for (int i = tid; i < WKV_LC * WKV_CW; i += 256) {
      const int t = i / WKV_CW, x = i - t * WKV_CW;
      vs[i] = (t < n && c0 + x < vdim) ? to_f32(vv[(long long)(b0 + t) * ldv + h * vdim + c0 + x]) : 0.f;
    }
    __syncthreads();
    const bool live = c0 + col < vdim;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    // (unrolled by 4: unrolled whole, the 32 turns' loads and eight sums a thread run twice as slow)
#pragma unroll 4
    for (int j = 0; j < WKV_LC; ++j) {
      const float v = vs[j * WKV_CW + col];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(as[(tq + 4 * i) * (WKV_LC + 1) + j], v, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = tq + 4 * i;
      if (live && t < n) out[(long long)(b0 + t) * heads * vdim + h * vdim + c0 + col] = acc[i];
    }
    for (int cb = 0; cb < dim; cb += 32) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll 4
      for (int j = 0; j < WKV_LC; ++j) {
        const float v = vs[j * WKV_CW + col];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int c = cb + tq + 4 * i;
          acc[i] = fmaf(c < dim ? ks[j * ld + c] : 0.f, v, acc[i]);
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int c = cb + tq + 4 * i;
        if (live && c < dim) scratch[(((long long)ch * heads + h) * dim + c) * vdim + c0 + col] = acc[i];
      }
    }
  }
}

// grid (requests, heads, slices of the dim x vdim elements); req_chunks [requests + 1]: first chunk of each request
__global__ void __launch_bounds__(256)
wkv_scan_kernel(float* __restrict__ scratch, float* __restrict__ state, const float* __restrict__ dtot,
                const int* __restrict__ slot_ids, const int* __restrict__ req_chunks, int heads, int dim, int vdim) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int first = req_chunks[r], last = req_chunks[r + 1];
  if (last <= first) return;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= dim * vdim) return;
  const int c = e / vdim;
  float* S = state + ((long long)slot_ids[r] * heads + h) * dim * vdim + e;
  float s = *S;
  float next = scratch[((long long)first * heads + h) * dim * vdim + e];
  for (int ch = first; ch < last; ++ch) {
    float* U = scratch + ((long long)ch * heads + h) * dim * vdim + e;
    const float u = next;
    if (ch + 1 < last) next = U[(long long)heads * dim * vdim];     // asked for before this chunk's store
    *U = s;
    s = fmaf(dtot[((long long)ch * heads + h) * dim + c], s, u);
  }
  *S = s;
}

// grid (chunks, heads): out[t] += rq[t]^T S_before, S_before in scratch[chunk]
__global__ void __launch_bounds__(256)
wkv_apply_kernel(float* __restrict__ out, const float* __restrict__ scratch, const float* __restrict__ rq,
                 const int* __restrict__ work, const int* __restrict__ cu_seqlens, int heads, int dim, int vdim) {
  extern __shared__ float lds[];      // rq [LC][dim]
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int req = work[2 * ch], b0 = work[2 * ch + 1];
  const int n = min(WKV_LC, cu_seqlens[req + 1] - b0);
  for (int i = tid; i < WKV_LC * dim; i += 256) {
    const int t = i / dim, c = i - t * dim;
    lds[i] = t < n ? rq[(long long)(b0 + t) * heads * dim + h * dim + c] : 0.f;
  }
  __syncthreads();
  const int col = tid & (WKV_CW - 1), tq = tid / WKV_CW;
  for (int c0 = 0; c0 < vdim; c0 += WKV_CW) {
    if (c0 + col >= vdim) continue;
    const float* Sb = scratch + ((long long)ch * heads + h) * dim * vdim + c0 + col;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    for (int c = 0; c < dim; ++c) {
      const float s = Sb[(long long)c * vdim];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(lds[(tq + 4 * i) * dim + c], s, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = tq + 4 * i;
      if (t < n) out[(long long)(b0 + t) * heads * vdim + h * vdim + c0 + col] += acc[i];
    }
  }
}

extern "C" int jv_wkv_max_dim() { return WKV_ROWS * 256; }
extern "C" int jv_wkv_chunk_tokens() { return WKV_LC; }
extern "C" int jv_wkv_chunk_max_dim() { return 128; }

#define DEFINE_WKV(SUF, T)                                                                                      \
  extern "C" int jv_token_shift_mix_##SUF(void* out, const void* x, const float* mu, int n_mix, float* state,   \
                                          const int* slot_ids, const int* cu_seqlens, const int* token_req,     \
                                          long long n, int hidden, void* stream) {                              \
    if (n <= 0 || hidden <= 0 || n_mix <= 0) return 0;                                                          \
    if (n > 0x7fffffffll || (hidden + 255) / 256 > 65535) return (int)hipErrorInvalidValue;                     \
    constexpr int V = 16 / (int)sizeof(T);                                                                      \
    if (hidden % V == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)x % 16 == 0) {                                \
      hipLaunchKernelGGL(token_shift_mix_vec_kernel<T>, dim3((unsigned)n, (hidden / V + 255) / 256), dim3(256), \
                         0, (hipStream_t)stream, (T*)out, (const T*)x, mu, n_mix, state, slot_ids, cu_seqlens,  \
                         token_req, n, hidden);                                                                 \
      return JV_LAUNCH_CHECK();                                                                                 \
    }                                                                                                           \
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

// work [chunks][2] = (request, first token) in the order of requests and tokens, req_chunks [requests + 1]; scratch of
// chunks * heads * dim * vdim floats, rq of tokens * heads * dim floats, dtot of chunks * heads * dim floats.
#define DEFINE_WKV_CHUNKS(SUF, T)                                                                               \
  extern "C" int jv_wkv_chunks_##SUF(float* out, const void* r, long long ldr, const void* k, long long ldk,    \
                                     const void* v, long long ldv, const void* rate, long long ldw,             \
                                     const float* w0, const float* bonus, float* state, const int* slot_ids,    \
                                     const int* cu_seqlens, int n_requests, int heads, int dim, int vdim,       \
                                     int chunks, const int* work, const int* req_chunks, float* scratch,        \
                                     float* rq, float* dtot, void* stream) {                                    \
    if (n_requests <= 0 || heads <= 0 || chunks <= 0) return 0;                                                 \
    if (dim <= 0 || dim > 128 || vdim <= 0 || heads > 65535 || !work || !req_chunks || !scratch || !rq || !dtot) \
      return (int)hipErrorInvalidValue;                                                                         \
    if (((long long)dim * vdim + 255) / 256 > 65535) return (int)hipErrorInvalidValue;                          \
    hipStream_t s = (hipStream_t)stream;                                                                        \
    const size_t lds_local = (3 * WKV_LC * (dim + 1) + WKV_LC * (WKV_LC + 1) + WKV_LC * WKV_CW + dim) * sizeof(float); \
    hipLaunchKernelGGL(wkv_local_kernel<T>, dim3(chunks, heads), dim3(256), lds_local, s, out, scratch, rq, dtot, \
                       (const T*)r, ldr, (const T*)k, ldk, (const T*)v, ldv, (const T*)rate, ldw, w0, bonus,    \
                       work, cu_seqlens, heads, dim, vdim);                                                     \
    hipLaunchKernelGGL(wkv_scan_kernel, dim3(n_requests, heads, (dim * vdim + 255) / 256), dim3(256), 0, s,     \
                       scratch, state, dtot, slot_ids, req_chunks, heads, dim, vdim);                           \
    hipLaunchKernelGGL(wkv_apply_kernel, dim3(chunks, heads), dim3(256), (size_t)WKV_LC * dim * sizeof(float),  \
                       s, out, scratch, rq, work, cu_seqlens, heads, dim, vdim);                                \
    return JV_LAUNCH_CHECK();                                                                                   \
  }

DEFINE_WKV_CHUNKS(bf16, bf16_t)
DEFINE_WKV_CHUNKS(f32, float)
DEFINE_WKV(bf16, bf16_t)
DEFINE_WKV(f32, float)
