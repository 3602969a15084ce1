// Attention input for heads whose key and value sizes differ, whose q/k norm spans the whole
// projection, or whose rows hold more than q, k and v: from a token's row that begins with
// [q: nq * dk | k: nkv * dk | v: nkv * dv] (plus an optional bias)
//   q, k  <- RMS norm over ALL of q's (k's) columns at once, times a weight of that size (one block a token),
//            or (per_head) over every head on its own, times a weight of dk elements shared by the heads, or none
//            (a wave a (token, head))
//   q, k  <- the first rot_dims elements of every head turned by the token's angles
//   q     <- q * (1 + coef * ln(floor((position + 1) / every) + 1))    (optional: a query temperature that grows with position)
//   v     <- v * v_scale;  the v heads begin at column v_off of the row (behind k, or AT k: values that are the keys as projected)
// and stored in the layout the paged attention kernels read, every head padded with zeros to one size
// Dp >= max(dk, dv): q rows [n][nq][Dp], key pages [pages][nkv][page_size][Dp], value pages transposed
// [pages][nkv][Dp][page_size].  Zero padding leaves every score and every output element as it is; the
// pad of the pages is never written and stays the zero the storage starts with.  Sums, norms and angles
// are float.  The first kernel: one block a token; its row is kept in LDS between the passes.
#include "common.h"
#include "v_pages_write.h"

template <typename T>
__global__ void __launch_bounds__(1024)
attn_prepare_wide_kernel(T* __restrict__ q_out, const T* __restrict__ qkv, long long ld,
                         const float* __restrict__ bias, const float* __restrict__ q_w,
                         const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin,
                         int rot_dims, const int* __restrict__ slot_mapping, T* __restrict__ k_pages,
                         T* __restrict__ v_pages, int page_size, int nq, int nkv, int dk, int dv, int dp,
                         float v_scale) {
  extern __shared__ float row[];          // q | k, after bias
  __shared__ float red[32];
  const long long t = blockIdx.x;
  const int qn = nq * dk, kn = nkv * dk, vn = nkv * dv;
  const T* x = qkv + t * ld;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < qn + kn; c += blockDim.x) {
    const float a = to_f32(x[c]) + (bias ? bias[c] : 0.f);
    row[c] = a;
    if (c < qn) sq = fmaf(a, a, sq); else sk = fmaf(a, a, sk);
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (q_w) {
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    inv_q = rsqrtf(sq / (float)qn + eps);
    inv_k = rsqrtf(sk / (float)kn + eps);
  } else {
    __syncthreads();
  }
  const int half = rot_dims / 2;
  const int sm = slot_mapping ? slot_mapping[t] : -1;
  const long long page = sm >= 0 ? sm / page_size : 0;
  const int slot = sm >= 0 ? sm % page_size : 0;
  // q and k heads: element i of a padded head
  const int heads = nq + nkv;
  for (int e = threadIdx.x; e < heads * dp; e += blockDim.x) {
    const int hd = e / dp, i = e - hd * dp;
    const bool is_q = hd < nq;
    float val = 0.f;
    if (i < dk) {
      const int c = is_q ? hd * dk + i : qn + (hd - nq) * dk + i;
      const float inv = is_q ? inv_q : inv_k;
      const float* wn = is_q ? q_w : k_w;
      const int wc = is_q ? c : c - qn;
      val = row[c] * inv * (wn ? wn[wc] : 1.f);
      if (i < rot_dims) {
        const int j = i < half ? i : i - half;
        const int co = i < half ? c + half : c - half;
        const float other = row[co] * inv * (wn ? wn[is_q ? co : co - qn] : 1.f);
        const float cs = cos_sin[t * rot_dims + j], sn = cos_sin[t * rot_dims + half + j];
        val = i < half ? val * cs - other * sn : val * cs + other * sn;
      }
    }
    if (is_q) {
      q_out[(t * nq + hd) * dp + i] = from_f32<T>(val);
    } else if (sm >= 0 && i < dk) {
      k_pages[((page * nkv + (hd - nq)) * page_size + slot) * dp + i] = from_f32<T>(val);
    }
  }
  if (sm >= 0) {
    for (int e = threadIdx.x; e < vn; e += blockDim.x) {
      const int hd = e / dv, i = e - hd * dv;
      const float val = (to_f32(x[qn + kn + e]) + (bias ? bias[qn + kn + e] : 0.f)) * v_scale;
      v_pages[((page * nkv + hd) * dp + i) * page_size + slot] = from_f32<T>(val);
    }
  }
}


// The same for a norm per head (or none): nothing ties a token's heads together, so a wave takes one (token, head),
// four heads a block, and a step of few tokens still fills many compute units.  Heads nq + nkv .. nq + 2 nkv - 1 are
// the v heads (left out with v_elsewhere: the tile writer of many tokens takes them).  The head is kept in LDS
// between its norm and its rotation (dk floats a wave).
template <typename T>
__global__ void __launch_bounds__(256)
attn_prepare_heads_kernel(T* __restrict__ q_out, const T* __restrict__ qkv, long long ld,
                          const float* __restrict__ bias, const float* __restrict__ q_w,
                          const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin,
                          int rot_dims, const int* __restrict__ slot_mapping, T* __restrict__ k_pages,
                          T* __restrict__ v_pages, int page_size, int nq, int nkv, int dk, int dv, int dp,
                          float v_scale, int v_elsewhere, long long v_off, const int* __restrict__ positions,
                          float qt_coef, int qt_every) {
  extern __shared__ float heads_lds[];     // [4 waves][dk]
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  float* buf = heads_lds + wid * dk;
  const long long t = blockIdx.x;
  const int head = blockIdx.y * 4 + wid;
  const int n_heads = nq + 2 * nkv;
  const bool live = head < n_heads;
  const bool is_q = live && head < nq, is_v = live && head >= nq + nkv, is_k = live && !is_q && !is_v;
  const int sm = slot_mapping ? slot_mapping[t] : -1;
  const bool store = sm >= 0 && k_pages != nullptr;
  const long long page = store ? sm / page_size : 0;
  const int slot = store ? sm % page_size : 0;
  const T* x = qkv + t * ld;
  if (is_v && store && !v_elsewhere) {
    const int kvh = head - nq - nkv;
    const long long c0 = v_off + (long long)kvh * dv;
    T* dst = v_pages + (page * nkv + kvh) * (long long)dp * page_size + slot;
    for (int i = lane; i < dv; i += JV_WAVE)
      dst[(long long)i * page_size] = from_f32<T>((to_f32(x[c0 + i]) + (bias ? bias[c0 + i] : 0.f)) * v_scale);
  }
  const bool work = is_q || (is_k && store);      // a k head that nobody will read is skipped
  const int c0 = (live && !is_v ? head : 0) * dk;
  const float* w = is_q ? q_w : k_w;
  float inv = 1.f;
  if (work) {
    float ss = 0.f;
    for (int i = lane; i < dk; i += JV_WAVE) {
      const float a = to_f32(x[c0 + i]) + (bias ? bias[c0 + i] : 0.f);
      buf[i] = a;
      ss = fmaf(a, a, ss);
    }
    if (w) inv = rsqrtf(wave_sum(ss) / (float)dk + eps);
  }
  __syncthreads();      // every wave arrives once: the head in LDS is readable by the wave's other lanes
  if (!work) return;
  const float temp = (is_q && positions) ? 1.f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.f) : 1.f;
  const int half = rot_dims / 2;
  T* dst = is_q ? q_out + (t * nq + head) * dp : k_pages + ((page * nkv + (head - nq)) * page_size + slot) * (long long)dp;
  for (int i = lane; i < (is_q ? dp : dk); i += JV_WAVE) {
    float val = 0.f;
    if (i < dk) {
      val = buf[i] * inv * (w ? w[i] : 1.f);
      if (i < rot_dims) {
        const int j = i < half ? i : i - half;
        const int io = i < half ? i + half : i - half;
        const float other = buf[io] * inv * (w ? w[io] : 1.f);
        const float cs = cos_sin[t * rot_dims + j], sn = cos_sin[t * rot_dims + half + j];
        val = i < half ? val * cs - other * sn : val * cs + other * sn;
      }
    }
    dst[i] = from_f32<T>(val * temp);
  }
}

// The q and k heads of many tokens, 16 bytes a lane: a head of dk elements takes dk / EP lanes (a power of two), a
// wave takes 64 / (dk / EP) (token, head) pairs, the sum of squares is reduced among a head's lanes, and the partner of
// a rotated piece (half the rotated size further on, or back) sits in another lane of the same head: no LDS, no
// barrier.  The v heads go through the tile writer.  Needs dk, dp, ld and half the rotated size to be multiples of
// EP = 16 bytes' elements.
template <typename T>
__global__ void __launch_bounds__(256)
attn_prepare_heads_vec_kernel(T* __restrict__ q_out, const T* __restrict__ qkv, long long ld,
                              const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
                              const float* __restrict__ cos_sin, int rot_dims, const int* __restrict__ slot_mapping,
                              T* __restrict__ k_pages, int page_size, long long n_items, int nq, int nkv, int dk,
                              int dp, int lph, const int* __restrict__ positions, float qt_coef, int qt_every) {
  constexpr int EP = 16 / (int)sizeof(T);
  typedef T tv __attribute__((ext_vector_type(EP)));
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  const int hpw = JV_WAVE / lph, walk = nq + nkv;
  long long item = ((long long)blockIdx.x * 4 + wid) * hpw + lane / lph;
  const bool live = item < n_items;
  if (!live) item = n_items - 1;               // idle lanes go along through the shuffles and store nothing
  const long long t = item / walk;
  const int head = (int)(item - t * walk);
  const bool is_q = head < nq;
  const int j = lane & (lph - 1), e0 = j * EP;
  const int sm = slot_mapping ? slot_mapping[t] : -1;
  const bool store = sm >= 0 && k_pages != nullptr;
  const tv xv = *(const tv*)(qkv + t * ld + (long long)head * dk + e0);
  const float* w = is_q ? q_w : k_w;
  float a[EP], ss = 0.f;
#pragma unroll
  for (int e = 0; e < EP; ++e) { a[e] = to_f32<T>(xv[e]); ss = fmaf(a[e], a[e], ss); }
  if (w) {
    for (int o = lph / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, JV_WAVE);
    const float inv = rsqrtf(ss / (float)dk + eps);
#pragma unroll
    for (int e = 0; e < EP; ++e) a[e] *= inv * w[e0 + e];
  }
  const int half = rot_dims / 2;
  const bool turns = e0 < rot_dims, low = e0 < half;
  const int partner = turns ? (low ? lane + half / EP : lane - half / EP) : lane;
  float b[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) b[e] = __shfl(a[e], partner, JV_WAVE);
  if (turns) {
    const float* cs = cos_sin + t * rot_dims + (low ? e0 : e0 - half);
#pragma unroll
    for (int e = 0; e < EP; ++e) {
      const float c = cs[e], sn = cs[half + e];
      a[e] = low ? a[e] * c - b[e] * sn : a[e] * c + b[e] * sn;
    }
  }
  if (!live || !(is_q || store)) return;
  const float temp = (is_q && positions) ? 1.f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.f) : 1.f;
  tv ov;
#pragma unroll
  for (int e = 0; e < EP; ++e) ov[e] = from_f32<T>(a[e] * temp);
  if (is_q) {
    T* dst = q_out + (t * nq + head) * dp;
    *(tv*)(dst + e0) = ov;
    tv zero;
#pragma unroll
    for (int e = 0; e < EP; ++e) zero[e] = from_f32<T>(0.f);
    for (int c = dk + e0; c < dp; c += lph * EP) *(tv*)(dst + c) = zero;
  } else {
    const long long page = sm / page_size;
    const int slot = sm - (int)page * page_size;
    *(tv*)(k_pages + ((page * nkv + (head - nq)) * page_size + slot) * (long long)dp + e0) = ov;
  }
}

#define DEFINE_ATTN_PREPARE(SUF, T)                                                                             \
  extern "C" int jv_attn_prepare_wide_##SUF(void* q_out, const void* qkv, long long ld, const float* bias,      \
                                            const float* q_w, const float* k_w, float eps,                      \
                                            const float* cos_sin, int rot_dims, const int* slot_mapping,        \
                                            void* k_pages, void* v_pages, int page_size, int n, int nq,         \
                                            int nkv, int dk, int dv, int dp, float v_scale, int per_head,       \
                                            long long v_off, const int* positions, float qt_coef, int qt_every, \
                                            void* stream) {                                                     \
    if (n <= 0) return 0;                                                                                       \
    if (v_off < 0 || (positions && (qt_every <= 0 || (q_w && !per_head)))) return (int)hipErrorInvalidValue;    \
    if (q_w && !per_head && v_off != (long long)(nq + nkv) * dk) return (int)hipErrorInvalidValue;              \
    if (nq <= 0 || nkv <= 0 || dk <= 0 || dv <= 0 || dp < dk || dp < dv || rot_dims < 0 || rot_dims > dk ||     \
        rot_dims % 2 || (rot_dims && !cos_sin) || (!q_w) != (!k_w) || (slot_mapping && (!k_pages || !v_pages))) \
      return (int)hipErrorInvalidValue;                                                                         \
    if (!q_w || per_head) {                                                                                     \
      /* a wave a (token, head); the v heads of many tokens through the tile writer where its pieces align */  \
      constexpr int EP = 16 / (int)sizeof(T);                                                                   \
      const bool v_tile = slot_mapping && !bias && v_written_by_tile<T>(k_pages, n, page_size, dv) &&           \
                          ld % EP == 0 && v_off % EP == 0 && ((uintptr_t)qkv % 16) == 0;                        \
      if (v_tile) {                                                                                             \
        const int e = launch_v_pages_write<T>(qkv, ld, v_off, slot_mapping, v_pages, page_size, n, nkv, dv,     \
                                              dp, v_scale, stream);                                             \
        if (e) return e;                                                                                        \
      }                                                                                                         \
      const int lph = dk / EP;                                                                                  \
      if (v_tile && dk % EP == 0 && lph <= JV_WAVE && (lph & (lph - 1)) == 0 && dp % EP == 0 &&                 \
          (rot_dims / 2) % EP == 0 && (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_pages % 16 == 0) {             \
        const long long items = (long long)n * (nq + nkv);                                                      \
        const long long blocks = (items + 4 * (JV_WAVE / lph) - 1) / (4 * (JV_WAVE / lph));                     \
        if (blocks > 0x7fffffffll) return (int)hipErrorInvalidValue;                                            \
        hipLaunchKernelGGL(attn_prepare_heads_vec_kernel<T>, dim3((unsigned)blocks), dim3(256), 0,              \
                           (hipStream_t)stream, (T*)q_out, (const T*)qkv, ld, q_w, k_w, eps, cos_sin, rot_dims, \
                           slot_mapping, (T*)k_pages, page_size, items, nq, nkv, dk, dp, lph, positions,        \
                           qt_coef, qt_every);                                                                  \
        return JV_LAUNCH_CHECK();                                                                               \
      }                                                                                                         \
      const int walk = (v_tile || !slot_mapping) ? nq + nkv : nq + 2 * nkv;                                     \
      if ((walk + 3) / 4 > 65535 || (size_t)4 * dk * sizeof(float) > 64 * 1024) return (int)hipErrorInvalidValue; \
      hipLaunchKernelGGL(attn_prepare_heads_kernel<T>, dim3(n, (walk + 3) / 4), dim3(256),                      \
                         (size_t)4 * dk * sizeof(float), (hipStream_t)stream, (T*)q_out, (const T*)qkv, ld,     \
                         bias, q_w, k_w, eps, cos_sin, rot_dims, slot_mapping, (T*)k_pages, (T*)v_pages,        \
                         page_size, nq, nkv, dk, dv, dp, v_scale, v_tile ? 1 : 0, v_off, positions, qt_coef,   \
                         qt_every);                                                                             \
      return JV_LAUNCH_CHECK();                                                                                 \
    }                                                                                                           \
    const size_t shmem = (size_t)(nq + nkv) * dk * sizeof(float);                                               \
    if (shmem > 64 * 1024) return (int)hipErrorInvalidValue;                                                    \
    /* few tokens of many wide heads (a decode step): more threads a token */                                  \
    const int threads = (n <= 256 && (nq + nkv) * dp >= 4096) ? 1024 : 256;                                     \
    hipLaunchKernelGGL(attn_prepare_wide_kernel<T>, dim3(n), dim3(threads), shmem, (hipStream_t)stream, (T*)q_out, \
                       (const T*)qkv, ld, bias, q_w, k_w, eps, cos_sin, rot_dims, slot_mapping, (T*)k_pages,    \
                       (T*)v_pages, page_size, nq, nkv, dk, dv, dp, v_scale);                                   \
    return JV_LAUNCH_CHECK();                                                                                   \
  }

DEFINE_ATTN_PREPARE(bf16, bf16_t)
DEFINE_ATTN_PREPARE(f32, float)
