// Attention input for heads whose key and value sizes differ, whose q/k norm spans the whole
// projection, or whose rows hold more than q, k and v: from a token's row that begins with
// [q: nq * dk | k: nkv * dk | v: nkv * dv] (plus an optional bias)
//   q, k  <- RMS norm over ALL of q's (k's) columns at once, times a weight of that size (optional), or
//            (per_head) over every head on its own, times a weight of dk elements shared by the heads
//   q, k  <- the first rot_dims elements of every head turned by the token's angles
//   v     <- v * v_scale
// and stored in the layout the paged attention kernels read, every head padded with zeros to one size
// Dp >= max(dk, dv): q rows [n][nq][Dp], key pages [pages][nkv][page_size][Dp], value pages transposed
// [pages][nkv][Dp][page_size].  Zero padding leaves every score and every output element as it is; the
// pad of the pages is never written and stays the zero the storage starts with.  Sums, norms and angles
// are float.  One block a token; its row is kept in LDS between the passes.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(1024)
attn_prepare_wide_kernel(T* __restrict__ q_out, const T* __restrict__ qkv, long long ld,
                         const float* __restrict__ bias, const float* __restrict__ q_w,
                         const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin,
                         int rot_dims, const int* __restrict__ slot_mapping, T* __restrict__ k_pages,
                         T* __restrict__ v_pages, int page_size, int nq, int nkv, int dk, int dv, int dp,
                         float v_scale, int per_head) {
  extern __shared__ float row[];          // q | k, after bias; then (per_head) one inverse root per head
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
  float* inv_head = row + qn + kn;
  if (q_w && per_head) {
    __syncthreads();
    // a wave a head in turns; the sum over a head's elements in a fixed order
    const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE, nw = blockDim.x / JV_WAVE;
    for (int hd = wid; hd < nq + nkv; hd += nw) {
      float s = 0.f;
      for (int i = lane; i < dk; i += JV_WAVE) s = fmaf(row[hd * dk + i], row[hd * dk + i], s);
      s = wave_sum(s);
      if (lane == 0) inv_head[hd] = rsqrtf(s / (float)dk + eps);
    }
    __syncthreads();
  } else if (q_w) {
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
      const float inv = (q_w && per_head) ? inv_head[hd] : (is_q ? inv_q : inv_k);
      const float* wn = is_q ? q_w : k_w;
      const int wc = per_head ? i : (is_q ? c : c - qn);
      val = row[c] * inv * (wn ? wn[wc] : 1.f);
      if (i < rot_dims) {
        const int j = i < half ? i : i - half;
        const int co = i < half ? c + half : c - half;
        const int wo = per_head ? (i < half ? i + half : i - half) : (is_q ? co : co - qn);
        const float other = row[co] * inv * (wn ? wn[wo] : 1.f);
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

#define DEFINE_ATTN_PREPARE(SUF, T)                                                                             \
  extern "C" int jv_attn_prepare_wide_##SUF(void* q_out, const void* qkv, long long ld, const float* bias,      \
                                            const float* q_w, const float* k_w, float eps,                      \
                                            const float* cos_sin, int rot_dims, const int* slot_mapping,        \
                                            void* k_pages, void* v_pages, int page_size, int n, int nq,         \
                                            int nkv, int dk, int dv, int dp, float v_scale, int per_head,       \
                                            void* stream) {                                                     \
    if (n <= 0) return 0;                                                                                       \
    if (nq <= 0 || nkv <= 0 || dk <= 0 || dv <= 0 || dp < dk || dp < dv || rot_dims < 0 || rot_dims > dk ||     \
        rot_dims % 2 || (rot_dims && !cos_sin) || (!q_w) != (!k_w) || (slot_mapping && (!k_pages || !v_pages))) \
      return (int)hipErrorInvalidValue;                                                                         \
    const size_t shmem = (size_t)(nq + nkv) * (dk + 1) * sizeof(float);                                         \
    if (shmem > 64 * 1024) return (int)hipErrorInvalidValue;                                                    \
    /* few tokens of many wide heads (a decode step): more threads a token */                                  \
    const int threads = (n <= 256 && (nq + nkv) * dp >= 4096) ? 1024 : 256;                                     \
    hipLaunchKernelGGL(attn_prepare_wide_kernel<T>, dim3(n), dim3(threads), shmem, (hipStream_t)stream, (T*)q_out, \
                       (const T*)qkv, ld, bias, q_w, k_w, eps, cos_sin, rot_dims, slot_mapping, (T*)k_pages,    \
                       (T*)v_pages, page_size, nq, nkv, dk, dv, dp, v_scale, per_head);                         \
    return JV_LAUNCH_CHECK();                                                                                   \
  }

DEFINE_ATTN_PREPARE(bf16, bf16_t)
DEFINE_ATTN_PREPARE(f32, float)
