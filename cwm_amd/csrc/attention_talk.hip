// Paged causal attention whose heads exchange their softmax weights ("talking heads" after the softmax), with grouped
// key/value heads, an optional sliding window and an optional sink in every head's softmax denominator.
//
//   s_g(i, j) = scale * q_g(i) . k_c(g)(j)                     over the keys j the query at i reads (its own and the
//                                                              `window_left` before it; all if window_left < 0)
//   p_g(i, j) = exp(s_g(i, j)) / (sum_j' exp(s_g(i, j')) + exp(sink_g))
//   w_h(i, j) = sum_g talk[h, g] p_g(i, j)                     the heads' weights are mixed after the softmax
//   o_h(i)    = sum_j w_h(i, j) v_c(h)(j)                      head h applies its mixed weights to its own values
//
// The mixed weight of a head needs the finished softmax of every head over all keys, so the scores are written out,
// float32, and the work is three stages over a table of scores [rows][heads][columns] (a row is a token of the step,
// column j of a row is the key `base + j` of the row's sequence, `base` the first key that the sequence's first token
// of the step reads):
//   1. `talk_scores_kernel`: a block a (row, key/value head, range of TALK_SPLIT columns) stages tiles of keys in LDS
//      and leaves the scaled scores of the head's query heads;
//   2. `talk_stats_kernel` (a block a (row, head): maximum and normaliser with the sink, over the columns the row
//      may read) and `talk_mix_kernel` (a thread a column: every head's normalised weight, then the mixed weights,
//      written in the activation type; zero for a column the row does not read);
//   3. `talk_values_kernel`: a block a (row, key/value head, range of columns) adds weight times value and leaves a
//      partial sum a range, which the caller adds in their order (the weights are final, so the partial sums are plain).
// Every block reads only its own head's keys or values, once.  A long portion of a prompt in bfloat16 takes stages 1
// and 3 as matrix products on keys and values gathered from the pages (`talk_gather_kernel`), with the scores and
// weights of a sequence as [key/value head][row][head of the group][column]; stage 2 takes either layout by its
// strides.  Every sum's order depends only on the row's own position, its sequence's portion and the window.
// float32 arithmetic for either storage type.  A key whose page is missing gives NaN.
#include "common.h"

CWM_DEFINE_ERROR_API

#define TALK_THREADS 256
#define TALK_TILE 32      // keys of a tile
#define TALK_SPLIT 128    // columns of a block's range (a multiple of the tile)
#define TALK_MAX_HEADS 64
#define TALK_MAX_HEAD_DIM 256
#define TALK_MIX_COLUMNS 256  // columns of a block of the mixing kernel

extern "C" int cwm_talking_attention_split() { return TALK_SPLIT; }
extern "C" int cwm_talking_attention_max_heads() { return TALK_MAX_HEADS; }

// Which rows a launch works on and where they sit in their sequences.
struct TalkRows {
  const int* token_list;    // row -> token of the step (null: row r is token r)
  const int* positions;     // the step's vectors; null: the rows are one sequence's consecutive tokens,
  const int* seq_of_token;
  const int* cu_q;
  const int* kv_len;
  int pos0, base0;          // whose row r is position pos0 + r and whose columns count from key base0
  int window_left;
};

struct TalkRow {
  int token, p, base, seq, first;  // position, first column's key, sequence, first key the row reads
};

__device__ __forceinline__ TalkRow talk_row(const TalkRows& R, int r) {
  TalkRow row;
  if (!R.positions) {
    row.token = r, row.p = R.pos0 + r, row.base = R.base0, row.seq = 0;
  } else {
    row.token = R.token_list ? R.token_list[r] : r;
    row.p = R.positions[row.token];
    row.seq = R.seq_of_token[row.token];
    const int p_first = R.kv_len[row.seq] - (R.cu_q[row.seq + 1] - R.cu_q[row.seq]);
    row.base = R.window_left >= 0 ? max(0, p_first - R.window_left) : 0;
  }
  row.first = R.window_left >= 0 ? max(0, row.p - R.window_left) : 0;
  return row;
}

// Where the scores and weights of (row, head, column) lie: element = kv_head * stride_c + row * stride_r +
// head_of_group * stride_g + column.
struct TalkLayout {
  long stride_c, stride_r, stride_g;
  int columns;
};

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

struct TalkCache {
  int n_kv_heads, head_dim, page_size, num_pages, table_width;
};

// the pages of the tile's keys j0 .. j0 + n_keys - 1 into LDS
__device__ __forceinline__ void talk_pages(int* pages, const TalkCache& ch, const int* __restrict__ table_row, int j0, int n_keys) {
  if (threadIdx.x < TALK_TILE) {
    int page = -1;
    if ((int)threadIdx.x < n_keys) {
      const int lp = (j0 + threadIdx.x) / ch.page_size;
      page = lp < ch.table_width ? table_row[lp] : -1;
      if (page >= ch.num_pages) page = -1;
    }
    pages[threadIdx.x] = page;
  }
}

// ---- stage 1 -------------------------------------------------------------------------------------------------------- //
template <typename T>
__global__ void __launch_bounds__(TALK_THREADS)
talk_scores_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ cache, const int* __restrict__ block_table,
                   float* __restrict__ scores, TalkRows R, TalkLayout L, TalkCache ch, int n_q_heads, float scale) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int hd = ch.head_dim, per = n_q_heads / ch.n_kv_heads;
  float* qs = lds;                                  // [per][hd]
  float* tile = qs + (size_t)per * hd;              // [TILE][hd + 1]
  int* pages = (int*)(tile + (size_t)TALK_TILE * (hd + 1));
  const int r = blockIdx.x, c = blockIdx.y, split = blockIdx.z;
  const TalkRow row = talk_row(R, r);
  // the row's keys among this block's columns: [k0, k1)
  const int k0 = max(row.first, row.base + split * TALK_SPLIT);
  const int k1 = min(row.p + 1, row.base + (split + 1) * TALK_SPLIT);
  if (k0 >= k1) return;  // the row reads none of them: nobody reads these scores
  const int* table_row = block_table + (size_t)row.seq * ch.table_width;
  const bool vec = hd % TalkVec<T>::N == 0 && ((uintptr_t)cache % 16) == 0;
  const size_t plane = (size_t)ch.n_kv_heads * ch.page_size * hd;
  const float nan = __uint_as_float(0x7fc00000u);
  const T* qrow = q + (size_t)row.token * q_stride + (size_t)c * per * hd;
  for (int e = threadIdx.x; e < per * hd; e += TALK_THREADS) qs[e] = Elem<T>::load(qrow + e);
  // lanes that share a dot product: so many that the (head, key) pairs of a tile fill the block
  int dsplit = 1;
  while (dsplit < 8 && per * TALK_TILE * dsplit * 2 <= TALK_THREADS) dsplit *= 2;
  float* out = scores + (size_t)c * L.stride_c + (size_t)r * L.stride_r - row.base;  // + head * stride_g + key
  for (int j0 = k0 - k0 % 8; j0 < k1; j0 += TALK_TILE) {
    const int n_keys = min(TALK_TILE, k1 - j0);
    __syncthreads();  // the tile and the pages of the round before have been read
    talk_pages(pages, ch, table_row, j0, n_keys);
    __syncthreads();
    if (vec) {
      constexpr int N = TalkVec<T>::N;
      const int pieces = hd / N;
      for (int e = threadIdx.x; e < n_keys * pieces; e += TALK_THREADS) {
        const int j = e / pieces, d0 = N * (e - j * pieces);
        const int page = pages[j];
        const int slot = (j0 + j) % ch.page_size;
        float v[N];
        if (page >= 0 && j0 + j >= k0) {
          TalkVec<T>::load(cache + (size_t)page * 2 * plane + ((size_t)c * ch.page_size + slot) * hd + d0, v);
        } else {
#pragma unroll
          for (int i = 0; i < N; ++i) v[i] = nan;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) tile[j * (hd + 1) + d0 + i] = v[i];
      }
    } else {
      for (int e = threadIdx.x; e < n_keys * hd; e += TALK_THREADS) {
        const int j = e / hd, d = e - j * hd;
        const int page = pages[j];
        const int slot = (j0 + j) % ch.page_size;
        float v = nan;
        if (page >= 0 && j0 + j >= k0) v = Elem<T>::load(cache + (size_t)page * 2 * plane + ((size_t)c * ch.page_size + slot) * hd + d);
        tile[j * (hd + 1) + d] = v;
      }
    }
    __syncthreads();
    // every thread takes part in the shuffles; the pairs beyond the last are computed and dropped
    const int items = per * TALK_TILE * dsplit;
    for (int e0 = 0; e0 < items; e0 += TALK_THREADS) {
      const int e = e0 + threadIdx.x;
      const int part = e % dsplit, pair = min(e / dsplit, per * TALK_TILE - 1);
      const int gl = pair / TALK_TILE, j = pair - gl * TALK_TILE;
      const bool counts = j < n_keys && j0 + j >= k0;
      float dot = 0.f;
      if (counts) {
        const float* qr = qs + (size_t)gl * hd;
        const float* kr = tile + (size_t)j * (hd + 1);
        float a0 = 0.f, a1 = 0.f;
        int d = part;
        for (; d + dsplit < hd; d += 2 * dsplit) a0 = fmaf(qr[d], kr[d], a0), a1 = fmaf(qr[d + dsplit], kr[d + dsplit], a1);
        if (d < hd) a0 = fmaf(qr[d], kr[d], a0);
        dot = a0 + a1;
      }
      for (int off = 1; off < dsplit; off *= 2) dot += __shfl_xor(dot, off, CWM_WAVE);
      if (part == 0 && e < items && counts) out[(size_t)gl * L.stride_g + j0 + j] = dot * scale;
    }
  }
}

// ---- stage 2 -------------------------------------------------------------------------------------------------------- //
// stats: [rows][heads][2]: the maximum (the sink included) and the inverse of the normaliser.  A block of four
// wavefronts a (row, head), whatever the number of columns: the order of the sums hangs on the row alone.
#define TALK_STATS_THREADS 256
__global__ void __launch_bounds__(TALK_STATS_THREADS)
talk_stats_kernel(const float* __restrict__ scores, float* __restrict__ stats, const float* __restrict__ sink, TalkRows R,
                  TalkLayout L, int n_q_heads, int per, float score_scale) {
  __shared__ float scratch[16];
  const int r = blockIdx.x, g = blockIdx.y;
  const TalkRow row = talk_row(R, r);
  const float* s = scores + (size_t)(g / per) * L.stride_c + (size_t)r * L.stride_r + (size_t)(g % per) * L.stride_g - row.base;
  float m = -__builtin_inff();
  for (int j = row.first + threadIdx.x; j <= row.p; j += TALK_STATS_THREADS) m = fmaxf(m, s[j] * score_scale);
  m = block_max(m, scratch);
  if (sink) m = fmaxf(m, sink[g]);
  float l = 0.f;
  for (int j = row.first + threadIdx.x; j <= row.p; j += TALK_STATS_THREADS) l += __expf(s[j] * score_scale - m);  // a NaN among the scores stays
  l = block_sum(l, scratch);
  if (sink) l += __expf(sink[g] - m);
  if (threadIdx.x == 0) {
    stats[((size_t)r * n_q_heads + g) * 2] = m;
    stats[((size_t)r * n_q_heads + g) * 2 + 1] = 1.0f / l;
  }
}

// weights: the layout of the scores, of TW; zero in the columns (below L.columns) that a row does not read
template <typename TW>
__global__ void __launch_bounds__(TALK_MIX_COLUMNS)
talk_mix_kernel(const float* __restrict__ scores, const float* __restrict__ stats, const float* __restrict__ talk,
                TW* __restrict__ weights, TalkRows R, TalkLayout L, int n_q_heads, int per, float score_scale) {
  extern __shared__ __attribute__((aligned(16))) float probs[];  // [heads][TALK_MIX_COLUMNS]
  const int r = blockIdx.x;
  const int col = blockIdx.y * TALK_MIX_COLUMNS + threadIdx.x;
  const TalkRow row = talk_row(R, r);
  const int key = row.base + col;
  const bool reads = col < L.columns && key >= row.first && key <= row.p;
  const size_t at = (size_t)r * L.stride_r + col;
  for (int g = 0; g < n_q_heads; ++g) {
    float p = 0.f;
    if (reads) {
      const float s = scores[(size_t)(g / per) * L.stride_c + (size_t)(g % per) * L.stride_g + at] * score_scale;
      p = __expf(s - stats[((size_t)r * n_q_heads + g) * 2]) * stats[((size_t)r * n_q_heads + g) * 2 + 1];
    }
    probs[g * TALK_MIX_COLUMNS + threadIdx.x] = p;  // a thread reads back only what it wrote itself
  }
  if (col >= L.columns) return;
  for (int h = 0; h < n_q_heads; ++h) {
    float w;
    if (talk) {
      w = 0.f;
      const float* trow = talk + (size_t)h * n_q_heads;  // the same address for the whole block
      for (int g = 0; g < n_q_heads; ++g) w = fmaf(trow[g], probs[g * TALK_MIX_COLUMNS + threadIdx.x], w);
    } else {
      w = probs[h * TALK_MIX_COLUMNS + threadIdx.x];
    }
    Elem<TW>::store(weights + (size_t)(h / per) * L.stride_c + (size_t)(h % per) * L.stride_g + at, reads ? w : 0.f);
  }
}

// ---- stage 3 -------------------------------------------------------------------------------------------------------- //
// NACC: output elements a thread adds up (heads of a group * head_dim <= NACC * TALK_THREADS).
// partial: float32 [ranges][rows][heads * head_dim]; a range that the row does not read leaves zeros.
template <typename T, typename TW, int NACC>
__global__ void __launch_bounds__(TALK_THREADS)
talk_values_kernel(const TW* __restrict__ weights, const T* __restrict__ cache, const int* __restrict__ block_table,
                   float* __restrict__ partial, TalkRows R, TalkLayout L, TalkCache ch, int n_q_heads, int n_rows) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int hd = ch.head_dim, per = n_q_heads / ch.n_kv_heads;
  float* wt = lds;                                   // [per][TILE]
  float* tile = wt + (size_t)per * TALK_TILE;        // [TILE][hd + 1]
  int* pages = (int*)(tile + (size_t)TALK_TILE * (hd + 1));
  const int r = blockIdx.x, c = blockIdx.y, split = blockIdx.z;
  const TalkRow row = talk_row(R, r);
  const int k0 = max(row.first, row.base + split * TALK_SPLIT);
  const int k1 = min(row.p + 1, row.base + (split + 1) * TALK_SPLIT);
  float acc[NACC];
#pragma unroll
  for (int n = 0; n < NACC; ++n) acc[n] = 0.f;
  if (k0 < k1) {
    const int* table_row = block_table + (size_t)row.seq * ch.table_width;
    const size_t plane = (size_t)ch.n_kv_heads * ch.page_size * hd;
    const int v_block = (ch.page_size % 8 == 0) ? 8 : ch.page_size;
    const bool vec_v = v_block == 8 && ((uintptr_t)cache % 16) == 0;
    const float nan = __uint_as_float(0x7fc00000u);
    const T* vplane = cache + plane + (size_t)c * hd * ch.page_size;
    const TW* w = weights + (size_t)c * L.stride_c + (size_t)r * L.stride_r - row.base;
    for (int j0 = k0 - k0 % 8; j0 < k1; j0 += TALK_TILE) {
      const int n_keys = min(TALK_TILE, k1 - j0);
      __syncthreads();  // the tile, the weights and the pages of the round before have been read
      talk_pages(pages, ch, table_row, j0, n_keys);
      for (int e = threadIdx.x; e < per * TALK_TILE; e += TALK_THREADS) {
        const int gl = e / TALK_TILE, j = e - gl * TALK_TILE;
        wt[e] = (j < n_keys && j0 + j >= k0) ? Elem<TW>::load(w + (size_t)gl * L.stride_g + j0 + j) : 0.f;
      }
      __syncthreads();
      if (vec_v) {
        // a block of 8 consecutive keys of one dimension is 8 consecutive elements: [slot / 8][dim][slot % 8]
        const int blocks = (n_keys + 7) / 8;
        for (int e = threadIdx.x; e < blocks * hd; e += TALK_THREADS) {
          const int jb = e / hd, d = e - jb * hd;
          const int page = pages[jb * 8];
          const int slot = (j0 + jb * 8) % ch.page_size;
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
            if (j < n_keys) tile[j * (hd + 1) + d] = (j0 + j >= k0) ? v[i] : 0.f;  // a key that does not count has weight zero
          }
        }
      } else {
        for (int e = threadIdx.x; e < n_keys * hd; e += TALK_THREADS) {
          const int j = e / hd, d = e - j * hd;
          const int page = pages[j];
          const int slot = (j0 + j) % ch.page_size;
          float v = 0.f;
          if (j0 + j >= k0) {
            v = nan;
            if (page >= 0) v = Elem<T>::load(vplane + (size_t)page * 2 * plane + ((size_t)(slot / v_block) * hd + d) * v_block + slot % v_block);
          }
          tile[j * (hd + 1) + d] = v;
        }
      }
      __syncthreads();
#pragma unroll
      for (int n = 0; n < NACC; ++n) {
        const int e = threadIdx.x + n * TALK_THREADS;
        if (e < per * hd) {
          const int gl = e / hd, d = e - gl * hd;
          const float* wrow = wt + gl * TALK_TILE;
          float a = acc[n];
          for (int j = 0; j < n_keys; ++j) a = fmaf(wrow[j], tile[j * (hd + 1) + d], a);
          acc[n] = a;
        }
      }
    }
  }
  float* dst = partial + ((size_t)split * n_rows + r) * n_q_heads * hd + (size_t)c * per * hd;
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = threadIdx.x + n * TALK_THREADS;
    if (e < per * hd) dst[e] = acc[n];
  }
}

// ---- keys and values of one sequence, gathered from its pages ------------------------------------------------------- //
// keys, values: [n_kv_heads][n_keys][head_dim], key j the sequence's key first + j
template <typename T>
__global__ void __launch_bounds__(TALK_THREADS)
talk_gather_kernel(const T* __restrict__ cache, const int* __restrict__ table_row, T* __restrict__ keys, T* __restrict__ values,
                   TalkCache ch, int first, int n_keys) {
  const int j = blockIdx.x, c = blockIdx.y, hd = ch.head_dim;
  const int key = first + j;
  const int lp = key / ch.page_size, slot = key % ch.page_size;
  int page = lp < ch.table_width ? table_row[lp] : -1;
  if (page >= ch.num_pages) page = -1;
  const size_t plane = (size_t)ch.n_kv_heads * ch.page_size * hd;
  const int v_block = (ch.page_size % 8 == 0) ? 8 : ch.page_size;
  const size_t at = page >= 0 ? (size_t)page * 2 * plane : 0;
  const T* kp = cache + at + ((size_t)c * ch.page_size + slot) * hd;
  const T* vp = cache + at + plane + (size_t)c * hd * ch.page_size + (size_t)(slot / v_block) * hd * v_block + slot % v_block;
  T* kd = keys + ((size_t)c * n_keys + j) * hd;
  T* vd = values + ((size_t)c * n_keys + j) * hd;
  const float nan = __uint_as_float(0x7fc00000u);
  for (int d = threadIdx.x; d < hd; d += blockDim.x) {
    Elem<T>::store(kd + d, page >= 0 ? Elem<T>::load(kp + d) : nan);
    Elem<T>::store(vd + d, page >= 0 ? Elem<T>::load(vp + (size_t)d * v_block) : nan);
  }
}

// ---- entry points ---------------------------------------------------------------------------------------------------- //
static inline int talk_check(int n_q_heads, int n_kv_heads, int head_dim, int page_size, int num_pages, int table_width) {
  CWM_REQUIRE(n_q_heads >= 1 && n_q_heads <= TALK_MAX_HEADS && n_kv_heads >= 1 && n_q_heads % n_kv_heads == 0,
              "talking_attention: %d query heads on %d key/value heads (at most %d heads)", n_q_heads, n_kv_heads, TALK_MAX_HEADS);
  CWM_REQUIRE(head_dim >= 1 && head_dim <= TALK_MAX_HEAD_DIM, "talking_attention: head size %d is outside 1..%d", head_dim, TALK_MAX_HEAD_DIM);
  CWM_REQUIRE(page_size >= 1 && num_pages >= 1 && table_width >= 1, "talking_attention: bad cache sizes");
  return 0;
}

// Stages 1 to 3 on rows of the step's tokens.  q: [T, H, hd] of `dtype` (tokens q_stride apart), as the paged cache
// [pages, 2, Hkv, page * hd] (keys [slot][dim]; values [slot / 8][dim][slot % 8], or the whole page as one block where
// the page size is no multiple of 8).  token_list: int32 [n_rows] or null (the rows are all n_rows tokens).  columns: of
// the score table, a multiple of TALK_SPLIT that holds every row's keys counted from its sequence's base.  scores:
// float32 [n_rows, H, columns]; weights: the same of `dtype`; stats: float32 [n_rows, H, 2]; partial: float32
// [columns / TALK_SPLIT, n_rows, H * hd], which the caller adds up over the ranges.  sink: float32 [H] or null; talk:
// float32 [H, H] or null.
extern "C" int cwm_talking_attention(const void* q, long q_stride, int dtype, const void* cache, const int* block_table,
                                     int table_width, const int* token_list, const int* positions, const int* seq_of_token,
                                     const int* cu_q, const int* kv_len, int n_rows, int n_q_heads, int n_kv_heads,
                                     int head_dim, int page_size, int num_pages, int window_left, float scale, const float* sink,
                                     const float* talk, int columns, float* scores, void* weights, float* stats, float* partial,
                                     hipStream_t stream) {
  if (talk_check(n_q_heads, n_kv_heads, head_dim, page_size, num_pages, table_width)) return 1;
  CWM_REQUIRE(n_rows >= 0 && columns >= TALK_SPLIT && columns % TALK_SPLIT == 0, "talking_attention: bad sizes");
  CWM_REQUIRE(q && cache && block_table && positions && seq_of_token && cu_q && kv_len && scores && weights && stats && partial,
              "talking_attention: arguments missing");
  const int per = n_q_heads / n_kv_heads;
  CWM_REQUIRE(per * head_dim <= 16 * TALK_THREADS, "talking_attention: %d heads of %d a key/value head are more than a block adds up", per, head_dim);
  const size_t lds1 = sizeof(float) * ((size_t)per * head_dim + (size_t)TALK_TILE * (head_dim + 1)) + sizeof(int) * TALK_TILE;
  const size_t lds3 = sizeof(float) * ((size_t)per * TALK_TILE + (size_t)TALK_TILE * (head_dim + 1)) + sizeof(int) * TALK_TILE;
  CWM_REQUIRE(lds1 <= 65536 && lds3 <= 65536, "talking_attention: %d heads of %d a key/value head need more LDS than a block has", per, head_dim);
  CWM_REQUIRE(columns / TALK_SPLIT <= 65535 && n_kv_heads <= 65535, "talking_attention: too many ranges of columns for one launch");
  if (n_rows == 0) return 0;
  const TalkRows R{token_list, positions, seq_of_token, cu_q, kv_len, 0, 0, window_left};
  const TalkLayout L{(long)per * columns, (long)n_q_heads * columns, (long)columns, columns};
  const TalkCache ch{n_kv_heads, head_dim, page_size, num_pages, table_width};
  const int ranges = columns / TALK_SPLIT;
  const dim3 grid(n_rows, n_kv_heads, ranges);
  const size_t lds2 = sizeof(float) * (size_t)n_q_heads * TALK_MIX_COLUMNS;
  const dim3 grid_mix(n_rows, (columns + TALK_MIX_COLUMNS - 1) / TALK_MIX_COLUMNS);
#define CWM_TALK_VALUES(T, NACC)                                                                                          \
  hipLaunchKernelGGL((talk_values_kernel<T, T, NACC>), grid, dim3(TALK_THREADS), lds3, stream, (const T*)weights,          \
                     (const T*)cache, block_table, partial, R, L, ch, n_q_heads, n_rows)
#define CWM_TALK(T)                                                                                                       \
  do {                                                                                                                    \
    hipLaunchKernelGGL((talk_scores_kernel<T>), grid, dim3(TALK_THREADS), lds1, stream, (const T*)q, q_stride,             \
                       (const T*)cache, block_table, scores, R, L, ch, n_q_heads, scale);                                  \
    hipLaunchKernelGGL(talk_stats_kernel, dim3(n_rows, n_q_heads), dim3(TALK_STATS_THREADS), 0, stream, scores, stats, sink, R, L,   \
                       n_q_heads, per, 1.0f);                                                                              \
    hipLaunchKernelGGL((talk_mix_kernel<T>), grid_mix, dim3(TALK_MIX_COLUMNS), lds2, stream, scores, stats, talk,          \
                       (T*)weights, R, L, n_q_heads, per, 1.0f);                                                           \
    if (per * head_dim <= TALK_THREADS) CWM_TALK_VALUES(T, 1);                                                             \
    else if (per * head_dim <= 4 * TALK_THREADS) CWM_TALK_VALUES(T, 4);                                                    \
    else CWM_TALK_VALUES(T, 16);                                                                                           \
  } while (0)
  if (dtype == CWM_F32) CWM_TALK(float);
  else if (dtype == CWM_BF16) CWM_TALK(bf16_t);
  else return cwm_fail("talking_attention: unknown element type %d", dtype);
#undef CWM_TALK
#undef CWM_TALK_VALUES
  return cwm_launch_status("talking_attention");
}

// Stage 2 alone, on the scores of one sequence's consecutive tokens as a matrix product left them: scores float32
// [Hkv][n_rows][H / Hkv][columns], unscaled (they are multiplied by `scale` here); row r is position pos0 + r, column j
// the key base + j.  weights: the same layout, of `w_dtype`.  stats: float32 [n_rows, H, 2] scratch.
extern "C" int cwm_talking_mix(const float* scores, void* weights, int w_dtype, float* stats, int n_rows, int columns,
                               int n_q_heads, int n_kv_heads, int pos0, int base, int window_left, float scale,
                               const float* sink, const float* talk, hipStream_t stream) {
  CWM_REQUIRE(n_q_heads >= 1 && n_q_heads <= TALK_MAX_HEADS && n_kv_heads >= 1 && n_q_heads % n_kv_heads == 0,
              "talking_mix: %d query heads on %d key/value heads (at most %d heads)", n_q_heads, n_kv_heads, TALK_MAX_HEADS);
  CWM_REQUIRE(n_rows >= 0 && columns >= 1 && pos0 >= 0 && base >= 0, "talking_mix: bad sizes");
  CWM_REQUIRE(base + columns > pos0 + n_rows - 1, "talking_mix: the columns end before the last row's own key");
  CWM_REQUIRE(scores && weights && stats, "talking_mix: arguments missing");
  if (n_rows == 0) return 0;
  const int per = n_q_heads / n_kv_heads;
  const TalkRows R{nullptr, nullptr, nullptr, nullptr, nullptr, pos0, base, window_left};
  const TalkLayout L{(long)n_rows * per * columns, (long)per * columns, (long)columns, columns};
  const size_t lds2 = sizeof(float) * (size_t)n_q_heads * TALK_MIX_COLUMNS;
  const dim3 grid_mix(n_rows, (columns + TALK_MIX_COLUMNS - 1) / TALK_MIX_COLUMNS);
  hipLaunchKernelGGL(talk_stats_kernel, dim3(n_rows, n_q_heads), dim3(TALK_STATS_THREADS), 0, stream, scores, stats, sink, R, L, n_q_heads, per, scale);
  if (w_dtype == CWM_F32)
    hipLaunchKernelGGL((talk_mix_kernel<float>), grid_mix, dim3(TALK_MIX_COLUMNS), lds2, stream, scores, stats, talk, (float*)weights, R, L, n_q_heads, per, scale);
  else if (w_dtype == CWM_BF16)
    hipLaunchKernelGGL((talk_mix_kernel<bf16_t>), grid_mix, dim3(TALK_MIX_COLUMNS), lds2, stream, scores, stats, talk, (bf16_t*)weights, R, L, n_q_heads, per, scale);
  else
    return cwm_fail("talking_mix: unknown element type %d", w_dtype);
  return cwm_launch_status("talking_mix");
}

// keys, values: [Hkv][n_keys][hd] of `dtype`, key j the key first + j of the sequence whose block table row is given
extern "C" int cwm_talking_gather(const void* cache, int dtype, const int* table_row, int table_width, void* keys, void* values,
                                  int n_kv_heads, int head_dim, int page_size, int num_pages, int first, int n_keys,
                                  hipStream_t stream) {
  CWM_REQUIRE(n_kv_heads >= 1 && head_dim >= 1 && page_size >= 1 && num_pages >= 1 && table_width >= 1 && first >= 0 && n_keys >= 0,
              "talking_gather: bad sizes");
  CWM_REQUIRE(n_keys == 0 || (long)(first + n_keys - 1) / page_size < table_width, "talking_gather: the block table ends before the last key");
  CWM_REQUIRE(cache && table_row && keys && values, "talking_gather: arguments missing");
  if (n_keys == 0) return 0;
  const TalkCache ch{n_kv_heads, head_dim, page_size, num_pages, table_width};
  const dim3 grid(n_keys, n_kv_heads);
  const int threads = head_dim <= 64 ? 64 : (head_dim < TALK_THREADS ? (head_dim + 63) / 64 * 64 : TALK_THREADS);
  if (dtype == CWM_F32)
    hipLaunchKernelGGL((talk_gather_kernel<float>), grid, dim3(threads), 0, stream, (const float*)cache, table_row, (float*)keys, (float*)values, ch, first, n_keys);
  else if (dtype == CWM_BF16)
    hipLaunchKernelGGL((talk_gather_kernel<bf16_t>), grid, dim3(threads), 0, stream, (const bf16_t*)cache, table_row, (bf16_t*)keys, (bf16_t*)values, ch, first, n_keys);
  else
    return cwm_fail("talking_gather: unknown element type %d", dtype);
  return cwm_launch_status("talking_gather");
}
