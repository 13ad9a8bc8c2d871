// Paged causal attention whose heads exchange their softmax weights ("talking heads" after the softmax), with grouped
// key/value heads, an optional sliding window and an optional sink in every head's softmax denominator.
//
//   s_g(i, j) = scale * q_g(i) . k_c(g)(j)                     over the keys j the query at i reads (its own and the
//                                                              `window_left` before it; all if window_left < 0)
//   p_g(i, j) = exp(s_g(i, j)) / (sum_j' exp(s_g(i, j')) + exp(sink_g))
//   w_h(i, j) = sum_g talk[h, g] p_g(i, j)                     the heads' weights are mixed after the softmax
//   o_h(i)    = sum_j w_h(i, j) v_c(h)(j)                      head h applies its mixed weights to its own values
//
// The mixed weight of a head needs the finished softmax of every head, so the work is two passes over a token's
// keys.  The first (`talk_stats_kernel`) leaves every head's maximum and sum of exponentials; the second
// (`talk_apply_kernel`) computes the scores again, normalises them, mixes them over the heads and adds the values
// up.  A token's keys are cut into ranges of TALK_SPLIT keys counted from the first key the token reads; a block
// takes one (token, range) with all heads, walks the range in tiles of TALK_TILE keys that it stages in LDS (keys of
// one key/value head at a time), and the ranges' results are plain partial sums (the normaliser is known before the
// second pass), which the caller adds in their order.  Every sum's order depends only on the token's own position
// and the window, so a token's result is the same bits whatever else is in the batch and however its sequence was cut.
// float32 arithmetic for either storage type.  A key whose page is missing gives NaN.
#include "common.h"

CWM_DEFINE_ERROR_API

#define TALK_THREADS 256
#define TALK_TILE 32      // keys of a tile
#define TALK_SPLIT 128    // keys of a range (a multiple of the tile)
#define TALK_MAX_HEADS 64
#define TALK_MAX_HEAD_DIM 256
#define TALK_LDS_LIMIT 65536

extern "C" int cwm_talking_attention_split() { return TALK_SPLIT; }
extern "C" int cwm_talking_attention_max_heads() { return TALK_MAX_HEADS; }

struct TalkShape {
  int n_q_heads, n_kv_heads, head_dim, page_size, num_pages, table_width, window_left;
  float scale;
};

// LDS of a block: q [H][hd], a tile of keys or values [TILE][hd + 1], scores [H][TILE], mixed weights [H][TILE],
// a page per key of the tile, and two numbers a head
static inline size_t talk_lds_bytes(int heads, int hd) {
  return sizeof(float) * ((size_t)heads * hd + (size_t)TALK_TILE * (hd + 1) + 2 * (size_t)heads * TALK_TILE + 2 * (size_t)heads) + sizeof(int) * TALK_TILE;
}

struct TalkLds {
  float *q, *tile, *scores, *mixed, *head_a, *head_b;
  int* pages;
  __device__ TalkLds(float* base, int heads, int hd) {
    q = base;
    tile = q + (size_t)heads * hd;
    scores = tile + (size_t)TALK_TILE * (hd + 1);
    mixed = scores + (size_t)heads * TALK_TILE;
    head_a = mixed + (size_t)heads * TALK_TILE;
    head_b = head_a + heads;
    pages = (int*)(head_b + heads);
  }
};

// the token's keys that this block reads: [k0, k1)
__device__ __forceinline__ bool talk_range(int p, int window_left, int split, int& k0, int& k1) {
  const int first = window_left >= 0 ? max(0, p - window_left) : 0;
  k0 = first + split * TALK_SPLIT;
  k1 = min(p + 1, k0 + TALK_SPLIT);
  return k0 < k1;
}

template <typename T> struct TalkVec;
template <> struct TalkVec<bf16_t> {
  static constexpr int N = 8;  // elements of a 16-byte load
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 x = *(const uint4*)p;
    v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
    v[4] = __uint_as_float(x.z << 16), v[5] = __uint_as_float(x.z & 0xffff0000u);
    v[6] = __uint_as_float(x.w << 16), v[7] = __uint_as_float(x.w & 0xffff0000u);
  }
};
template <> struct TalkVec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  }
};

// The tile of TALK_TILE keys from j0 on (j0 a multiple of 8; the keys outside [k0, k1) do not count): their pages,
// then the scores of all heads against them, scores[g][j], -inf for a key that does not count.  `vec`: rows of keys can
// be read 16 bytes at a time.
template <typename T>
__device__ __forceinline__ void talk_scores(const TalkLds& s, const TalkShape& sh, const T* __restrict__ cache,
                                            const int* __restrict__ table_row, int j0, int k0, int k1, bool vec) {
  const int hd = sh.head_dim, per = sh.n_q_heads / sh.n_kv_heads;
  const size_t plane = (size_t)sh.n_kv_heads * sh.page_size * hd;
  const int n_keys = min(TALK_TILE, k1 - j0);
  const float nan = __uint_as_float(0x7fc00000u);
  __syncthreads();  // whoever still reads the tile, the scores or the pages of the round before is done
  if (threadIdx.x < TALK_TILE) {
    int page = -1;
    if ((int)threadIdx.x < n_keys) {
      const int lp = (j0 + threadIdx.x) / sh.page_size;
      page = lp < sh.table_width ? table_row[lp] : -1;
      if (page >= sh.num_pages) page = -1;
    }
    s.pages[threadIdx.x] = page;
  }
  // lanes that share a dot product: so many that a key/value head's (head, key) pairs fill the block
  int dsplit = 1;
  while (dsplit < 8 && per * TALK_TILE * dsplit * 2 <= TALK_THREADS) dsplit *= 2;
  for (int c = 0; c < sh.n_kv_heads; ++c) {
    __syncthreads();  // pages known; the tile of the head before has been read
    if (vec) {
      constexpr int N = TalkVec<T>::N;
      const int pieces = hd / N;
      for (int e = threadIdx.x; e < n_keys * pieces; e += TALK_THREADS) {
        const int j = e / pieces, d0 = N * (e - j * pieces);
        const int page = s.pages[j];
        const int slot = (j0 + j) % sh.page_size;
        float v[N];
        if (page >= 0 && j0 + j >= k0) {
          TalkVec<T>::load(cache + (size_t)page * 2 * plane + ((size_t)c * sh.page_size + slot) * hd + d0, v);
        } else {
#pragma unroll
          for (int i = 0; i < N; ++i) v[i] = nan;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) s.tile[j * (hd + 1) + d0 + i] = v[i];
      }
    } else {
      for (int e = threadIdx.x; e < n_keys * hd; e += TALK_THREADS) {
        const int j = e / hd, d = e - j * hd;
        const int page = s.pages[j];
        const int slot = (j0 + j) % sh.page_size;
        float v = nan;
        if (page >= 0 && j0 + j >= k0) v = Elem<T>::load(cache + (size_t)page * 2 * plane + ((size_t)c * sh.page_size + slot) * hd + d);
        s.tile[j * (hd + 1) + d] = v;
      }
    }
    __syncthreads();
    // every thread takes part in the shuffles; the pairs beyond the last are computed and dropped
    const int items = per * TALK_TILE * dsplit;
    for (int e0 = 0; e0 < items; e0 += TALK_THREADS) {
      const int e = e0 + threadIdx.x;
      const int part = e % dsplit, pair = min(e / dsplit, per * TALK_TILE - 1);
      const int gl = pair / TALK_TILE, j = pair - gl * TALK_TILE;
      const int g = c * per + gl;
      const bool counts = j < n_keys && j0 + j >= k0;
      float dot = 0.f;
      if (counts) {
        const float* qrow = s.q + (size_t)g * hd;
        const float* krow = s.tile + (size_t)j * (hd + 1);
        float a0 = 0.f, a1 = 0.f;
        int d = part;
        for (; d + dsplit < hd; d += 2 * dsplit) a0 = fmaf(qrow[d], krow[d], a0), a1 = fmaf(qrow[d + dsplit], krow[d + dsplit], a1);
        if (d < hd) a0 = fmaf(qrow[d], krow[d], a0);
        dot = a0 + a1;
      }
      for (int off = 1; off < dsplit; off *= 2) dot += __shfl_xor(dot, off, CWM_WAVE);
      if (part == 0 && e < items) s.scores[g * TALK_TILE + j] = counts ? dot * sh.scale : -__builtin_inff();
    }
  }
  __syncthreads();
}

template <typename T>
__device__ __forceinline__ void talk_load_q(const TalkLds& s, const T* __restrict__ qrow, int n) {
  for (int e = threadIdx.x; e < n; e += TALK_THREADS) s.q[e] = Elem<T>::load(qrow + e);
}

template <typename T>
__device__ __forceinline__ bool talk_rows_vec(const T* cache, int hd) {
  return hd % TalkVec<T>::N == 0 && ((uintptr_t)cache % 16) == 0;
}

// stats: [T, n_split, H, 2] (maximum, sum of exp(score - maximum)); a range without keys leaves (-inf, 0)
template <typename T>
__global__ void __launch_bounds__(TALK_THREADS)
talk_stats_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ cache, const int* __restrict__ block_table,
                  const int* __restrict__ positions, const int* __restrict__ seq_of_token, float* __restrict__ stats, TalkShape sh) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const TalkLds s(lds, sh.n_q_heads, sh.head_dim);
  const int t = blockIdx.x, split = blockIdx.y, heads = sh.n_q_heads;
  float* dst = stats + ((size_t)t * gridDim.y + split) * heads * 2;
  int k0, k1;
  if (!talk_range(positions[t], sh.window_left, split, k0, k1)) {
    for (int g = threadIdx.x; g < heads; g += TALK_THREADS) dst[2 * g] = -__builtin_inff(), dst[2 * g + 1] = 0.f;
    return;
  }
  const int* table_row = block_table + (size_t)seq_of_token[t] * sh.table_width;
  const bool vec = talk_rows_vec(cache, sh.head_dim);
  talk_load_q(s, q + (size_t)t * q_stride, heads * sh.head_dim);
  for (int g = threadIdx.x; g < heads; g += TALK_THREADS) s.head_a[g] = -__builtin_inff(), s.head_b[g] = 0.f;
  for (int j0 = k0 - k0 % 8; j0 < k1; j0 += TALK_TILE) {
    talk_scores(s, sh, cache, table_row, j0, k0, k1, vec);
    const int n_keys = min(TALK_TILE, k1 - j0);
    for (int g = threadIdx.x; g < heads; g += TALK_THREADS) {
      const float* row = s.scores + g * TALK_TILE;
      float m = s.head_a[g], l = s.head_b[g];
      float top = row[0];
      for (int j = 1; j < n_keys; ++j) top = fmaxf(top, row[j]);
      if (!(top <= m)) {  // a larger maximum (or NaN, which then stays)
        l *= __expf(m - top);  // exp(-inf) = 0 at the first tile
        m = top;
      }
      for (int j = 0; j < n_keys; ++j) l += __expf(row[j] - m);  // a key that does not count: exp(-inf) = 0
      s.head_a[g] = m, s.head_b[g] = l;
    }
  }
  __syncthreads();
  for (int g = threadIdx.x; g < heads; g += TALK_THREADS) dst[2 * g] = s.head_a[g], dst[2 * g + 1] = s.head_b[g];
}

// NACC: output elements a thread adds up (heads * head_dim <= NACC * TALK_THREADS).  `out`: [T, H * hd] of T where the
// launch has one range a token, else `partial`: float32 [n_split, T, H * hd], zeros for a range without keys.
template <typename T, int NACC>
__global__ void __launch_bounds__(TALK_THREADS)
talk_apply_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ cache, const int* __restrict__ block_table,
                  const int* __restrict__ positions, const int* __restrict__ seq_of_token, const float* __restrict__ stats,
                  const float* __restrict__ sink, const float* __restrict__ talk, T* __restrict__ out, float* __restrict__ partial,
                  int n_tokens, TalkShape sh) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const TalkLds s(lds, sh.n_q_heads, sh.head_dim);
  const int t = blockIdx.x, split = blockIdx.y, heads = sh.n_q_heads, hd = sh.head_dim;
  const int per = heads / sh.n_kv_heads, width = heads * hd;
  float acc[NACC];
#pragma unroll
  for (int n = 0; n < NACC; ++n) acc[n] = 0.f;
  int k0, k1;
  const int p = positions[t];
  if (talk_range(p, sh.window_left, split, k0, k1)) {
    const int* table_row = block_table + (size_t)seq_of_token[t] * sh.table_width;
    const bool vec = talk_rows_vec(cache, hd);
    talk_load_q(s, q + (size_t)t * q_stride, width);
    // every head's maximum and the inverse of its normaliser, over all ranges of the token, in their order
    const int first = sh.window_left >= 0 ? max(0, p - sh.window_left) : 0;
    const int n_split = (p - first) / TALK_SPLIT + 1;
    const bool short_launch = n_split > (int)gridDim.y;  // the caller gave fewer ranges than this token has: its row is NaN
    for (int g = threadIdx.x; g < heads; g += TALK_THREADS) {
      if (short_launch) {
        s.head_a[g] = __uint_as_float(0x7fc00000u), s.head_b[g] = 1.f;
        continue;
      }
      const float* st = stats + (size_t)t * gridDim.y * heads * 2 + 2 * g;
      float m = sink ? sink[g] : -__builtin_inff();
      for (int r = 0; r < n_split; ++r) m = fmaxf(m, st[(size_t)r * heads * 2]);
      float l = sink ? __expf(sink[g] - m) : 0.f;
      for (int r = 0; r < n_split; ++r) l += st[(size_t)r * heads * 2 + 1] * __expf(st[(size_t)r * heads * 2] - m);
      s.head_a[g] = m;
      s.head_b[g] = 1.0f / l;  // a NaN among the scores has made the sum NaN
    }
    const size_t plane = (size_t)sh.n_kv_heads * sh.page_size * hd;
    const int v_block = (sh.page_size % 8 == 0) ? 8 : sh.page_size;
    const bool vec_v = v_block == 8 && ((uintptr_t)cache % 16) == 0 && (hd * sizeof(T)) % 2 == 0;
    const float nan = __uint_as_float(0x7fc00000u);
    for (int j0 = k0 - k0 % 8; j0 < k1; j0 += TALK_TILE) {
      talk_scores(s, sh, cache, table_row, j0, k0, k1, vec);  // ends with a barrier: head_a, head_b are known too
      const int n_keys = min(TALK_TILE, k1 - j0);
      for (int e = threadIdx.x; e < heads * TALK_TILE; e += TALK_THREADS) {
        const int g = e / TALK_TILE, j = e - g * TALK_TILE;
        s.scores[e] = j < n_keys ? __expf(s.scores[e] - s.head_a[g]) * s.head_b[g] : 0.f;
      }
      __syncthreads();
      for (int e = threadIdx.x; e < heads * TALK_TILE; e += TALK_THREADS) {
        const int h = e / TALK_TILE, j = e - h * TALK_TILE;
        float w;
        if (talk) {
          w = 0.f;
          const float* trow = talk + (size_t)h * heads;
          for (int g = 0; g < heads; ++g) w = fmaf(trow[g], s.scores[g * TALK_TILE + j], w);
        } else {
          w = s.scores[e];
        }
        s.mixed[e] = w;
      }
      for (int c = 0; c < sh.n_kv_heads; ++c) {
        __syncthreads();  // the mixed weights are there; the tile of the head before has been read
        const T* vplane = cache + plane + (size_t)c * hd * sh.page_size;
        if (vec_v) {
          // a block of 8 consecutive keys of one dimension is 8 consecutive elements: [slot / 8][dim][slot % 8]
          const int blocks = (n_keys + 7) / 8;
          for (int e = threadIdx.x; e < blocks * hd; e += TALK_THREADS) {
            const int jb = e / hd, d = e - jb * hd;
            const int page = s.pages[jb * 8];
            const int slot = (j0 + jb * 8) % sh.page_size;
            float v[8];
            if (page >= 0) {
              const T* src = vplane + (size_t)page * 2 * plane + ((size_t)(slot / 8) * hd + d) * 8;
              if constexpr (TalkVec<T>::N == 8) {
                TalkVec<T>::load(src, v);
              } else {
                float a[4], b[4];
                TalkVec<T>::load(src, a);
                TalkVec<T>::load(src + 4, b);
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = a[i], v[4 + i] = b[i];
              }
            } else {
#pragma unroll
              for (int i = 0; i < 8; ++i) v[i] = nan;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const int j = jb * 8 + i;
              if (j < n_keys) s.tile[j * (hd + 1) + d] = (j0 + j >= k0) ? v[i] : 0.f;  // a key that does not count has weight zero
            }
          }
        } else {
          for (int e = threadIdx.x; e < n_keys * hd; e += TALK_THREADS) {
            const int j = e / hd, d = e - j * hd;
            const int page = s.pages[j];
            const int slot = (j0 + j) % sh.page_size;
            float v = 0.f;
            if (j0 + j >= k0) {
              v = nan;
              if (page >= 0) v = Elem<T>::load(vplane + (size_t)page * 2 * plane + ((size_t)(slot / v_block) * hd + d) * v_block + slot % v_block);
            }
            s.tile[j * (hd + 1) + d] = v;
          }
        }
        __syncthreads();
#pragma unroll
        for (int n = 0; n < NACC; ++n) {
          const int e = threadIdx.x + n * TALK_THREADS;
          if (e < width) {
            const int h = e / hd, d = e - h * hd;
            if (h / per == c) {
              const float* wrow = s.mixed + h * TALK_TILE;
              float a = acc[n];
              for (int j = 0; j < n_keys; ++j) a = fmaf(wrow[j], s.tile[j * (hd + 1) + d], a);
              acc[n] = a;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = threadIdx.x + n * TALK_THREADS;
    if (e < width) {
      if (partial)
        partial[((size_t)split * n_tokens + t) * width + e] = acc[n];
      else
        Elem<T>::store(out + (size_t)t * width + e, acc[n]);
    }
  }
}

// q: [T, H, hd] (tokens q_stride elements apart) of `dtype`, as the paged cache [pages, 2, Hkv, page * hd] (keys
// [slot][dim]; values [slot / 8][dim][slot % 8], or the whole page as one block where the page size is no multiple
// of 8).  sink: float32 [H] or null; talk: float32 [H, H] or null (no mixing).  n_split: ranges of TALK_SPLIT keys
// that the launch gives every token (at least what the token with the most keys needs).  stats: float32
// [T * n_split * H * 2] scratch.  n_split == 1: the result goes to `out` [T, H * hd]; else to `partial`, float32
// [n_split, T, H * hd], which the caller adds up.
extern "C" int cwm_talking_attention(const void* q, long q_stride, void* out, float* partial, float* stats, const void* cache,
                                     int dtype, const int* block_table, int table_width, const int* positions,
                                     const int* seq_of_token, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                     int page_size, int num_pages, int window_left, float scale, const float* sink,
                                     const float* talk, int n_split, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_split >= 1, "talking_attention: bad sizes");
  CWM_REQUIRE(n_q_heads >= 1 && n_q_heads <= TALK_MAX_HEADS && n_kv_heads >= 1 && n_q_heads % n_kv_heads == 0,
              "talking_attention: %d query heads on %d key/value heads (at most %d heads)", n_q_heads, n_kv_heads, TALK_MAX_HEADS);
  CWM_REQUIRE(head_dim >= 1 && head_dim <= TALK_MAX_HEAD_DIM, "talking_attention: head size %d is outside 1..%d", head_dim, TALK_MAX_HEAD_DIM);
  CWM_REQUIRE(page_size >= 1 && num_pages >= 1 && table_width >= 1, "talking_attention: bad cache sizes");
  CWM_REQUIRE(q && cache && block_table && positions && seq_of_token && stats, "talking_attention: arguments missing");
  CWM_REQUIRE(n_split == 1 ? out != nullptr : partial != nullptr, "talking_attention: no place for the result");
  const size_t lds = talk_lds_bytes(n_q_heads, head_dim);
  CWM_REQUIRE(lds <= TALK_LDS_LIMIT, "talking_attention: %d heads of %d need %zu bytes of LDS, more than %d", n_q_heads, head_dim, lds, TALK_LDS_LIMIT);
  const int width = n_q_heads * head_dim;
  CWM_REQUIRE(width <= 64 * TALK_THREADS, "talking_attention: %d output elements a token are more than %d", width, 64 * TALK_THREADS);
  if (n_tokens == 0) return 0;
  TalkShape sh{n_q_heads, n_kv_heads, head_dim, page_size, num_pages, table_width, window_left, scale};
  const dim3 grid(n_tokens, n_split);
  float* part = n_split == 1 ? nullptr : partial;
#define CWM_TALK_APPLY(T, NACC)                                                                                          \
  hipLaunchKernelGGL((talk_apply_kernel<T, NACC>), grid, dim3(TALK_THREADS), lds, stream, (const T*)q, q_stride,          \
                     (const T*)cache, block_table, positions, seq_of_token, stats, sink, talk, (T*)out, part, n_tokens, sh)
#define CWM_TALK(T)                                                                                                      \
  do {                                                                                                                   \
    hipLaunchKernelGGL((talk_stats_kernel<T>), grid, dim3(TALK_THREADS), lds, stream, (const T*)q, q_stride,              \
                       (const T*)cache, block_table, positions, seq_of_token, stats, sh);                                 \
    if (width <= 4 * TALK_THREADS) CWM_TALK_APPLY(T, 4);                                                                  \
    else if (width <= 16 * TALK_THREADS) CWM_TALK_APPLY(T, 16);                                                           \
    else CWM_TALK_APPLY(T, 64);                                                                                           \
  } while (0)
  if (dtype == CWM_F32) CWM_TALK(float);
  else if (dtype == CWM_BF16) CWM_TALK(bf16_t);
  else return cwm_fail("talking_attention: unknown element type %d", dtype);
#undef CWM_TALK
#undef CWM_TALK_APPLY
  return cwm_launch_status("talking_attention");
}
