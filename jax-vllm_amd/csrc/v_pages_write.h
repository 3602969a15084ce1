// The writer of many tokens' v heads into transposed pages, shared by the attention-input kernels.
#pragma once
#include "common.h"

// The v heads of many tokens into their transposed pages [page][kv head][Dp][slot] (a head of D elements, a page
// head of Dp >= D: the pad is never written).  A token's v heads start `v_off` elements into its row of
// `row_stride` elements; `v_scale` multiplies the values.  Token by token
// every element would be a store of its own, 2 bytes every `page_size` elements; here a block takes
// 16 consecutive tokens of one kv head through LDS and writes, for every element of the head, 8
// tokens at once (16 bytes) wherever 8 consecutive tokens have 8 consecutive slots that start at a
// multiple of 8 (the usual case for a prompt), and element by element elsewhere.
template <typename T> struct alignas(16) Pack8 { T v[8]; };

template <typename T>
__global__ void __launch_bounds__(256) v_pages_write_kernel(
    const T* __restrict__ qkv, long long row_stride, long long v_off, const int* __restrict__ slot_mapping,
    T* __restrict__ v_pages, int page_size, int n_tokens, int nkv, int D, int Dp, float v_scale) {
  constexpr int EP = 16 / (int)sizeof(T);          // elements of a 16-byte piece
  extern __shared__ __attribute__((aligned(16))) unsigned char v_tile_mem[];
  T* tile = (T*)v_tile_mem;                        // [16][D + EP]
  const int LROW = D + EP;
  const int t0 = blockIdx.x * 16, kvh = blockIdx.y;
  const T* src = qkv + v_off + (long long)kvh * D;
  const int ppt = D / EP;
  for (int p = threadIdx.x; p < 16 * ppt; p += 256) {
    const int j = p / ppt, c = (p - j * ppt) * EP;
    if (t0 + j < n_tokens) *(uint4*)(tile + j * LROW + c) = *(const uint4*)(src + (t0 + j) * row_stride + c);
  }
  __syncthreads();
  for (int item = threadIdx.x; item < 2 * D; item += 256) {
    const int half = item / D, d = item - half * D;
    const int tb = t0 + half * 8;
    if (tb >= n_tokens) continue;
    const int s0 = slot_mapping[tb];
    bool run = s0 >= 0 && (s0 & 7) == 0 && tb + 8 <= n_tokens;
    if (run) {
#pragma unroll
      for (int j = 1; j < 8; ++j) run = run && slot_mapping[tb + j] == s0 + j;
    }
    const T* col = tile + (half * 8) * LROW + d;
    if (run) {
      const long long page = s0 / page_size;
      const int off = (int)(s0 - page * page_size);
      Pack8<T> v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v.v[j] = v_scale == 1.f ? col[j * LROW] : from_f32<T>(to_f32(col[j * LROW]) * v_scale);
      *(Pack8<T>*)(v_pages + ((page * nkv + kvh) * Dp + d) * (long long)page_size + off) = v;
    } else {
      for (int j = 0; j < 8 && tb + j < n_tokens; ++j) {
        const int s = slot_mapping[tb + j];
        if (s < 0) continue;
        const long long page = s / page_size;
        const int off = (int)(s - page * page_size);
        v_pages[((page * nkv + kvh) * Dp + d) * (long long)page_size + off] =
            v_scale == 1.f ? col[j * LROW] : from_f32<T>(to_f32(col[j * LROW]) * v_scale);
      }
    }
  }
}

// Whether the v heads of a step go through v_pages_write_kernel: many tokens, and sizes that keep
// its 16-byte pieces aligned (the caller also checks the row stride and the v heads' offset where they are its own).
template <typename T>
static bool v_written_by_tile(const void* k_pages, int n_tokens, int page_size, int D) {
  return k_pages != nullptr && n_tokens >= 256 && page_size % 8 == 0 && D % (16 / (int)sizeof(T)) == 0;
}

template <typename T>
static int launch_v_pages_write(const void* qkv, long long row_stride, long long v_off, const int* slot_mapping,
                                void* v_pages, int page_size, int n_tokens, int nkv, int D, int Dp, float v_scale,
                                void* stream) {
  if (nkv > 65535) return (int)hipErrorInvalidValue;
  const size_t shmem = (size_t)16 * (D + 16 / sizeof(T)) * sizeof(T);
  hipLaunchKernelGGL(v_pages_write_kernel<T>, dim3((n_tokens + 15) / 16, nkv), dim3(256), shmem,
                     (hipStream_t)stream, (const T*)qkv, row_stride, v_off, slot_mapping, (T*)v_pages, page_size,
                     n_tokens, nkv, D, Dp, v_scale);
  return JV_LAUNCH_CHECK();
}

