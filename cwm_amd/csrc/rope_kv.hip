// Rotary position encoding of queries and keys fused with the write of the new
// keys and values into the paged cache.
//
// Rotation (cwm/fastgen/kernels/rope.py:55-90): for pair i of a head,
//   a = float(pos) * inv_freq[i];  (x[2i], x[2i+1]) <- (x[2i] cos a - x[2i+1] sin a,
//                                                      x[2i+1] cos a + x[2i] sin a)
// in float32, the same for every head, applied to queries and keys and not to
// values, before the cache write (cwm/fastgen/forward.py:618-632).
//
// Cache layout of one layer: [num_pages][2][n_kv_heads][page_size * head_dim];
// plane 0 holds keys as [slot][dim]; plane 1 holds values in blocks of VB keys as
// [slot / VB][dim][slot % VB], VB = 8 if the page size is a multiple of 8 and the
// whole page otherwise, so that a matrix-core operand of the attention kernel (one
// dimension, 8 consecutive keys) is 16 contiguous bytes.  The row of a token is
// block_table[seq][pos / page_size], slot pos % page_size
// (cwm/fastgen/kernels/paged_memcpy.py:56-87 computes the same address).
#include "common.h"

CWM_DEFINE_ERROR_API

// bfloat16, head sizes of a multiple of 8: a thread takes four adjacent pairs (16 bytes) of a
// head, computes their four rotations once and applies them to that piece of every head of
// the token; keys go to the cache in the same 16-byte pieces.  Values: as in the kernel below.
// PARTIALS: q, k and v are not read but made here, from the float32 partial sums
// partials[p][t][q heads | k heads | v heads] of the joined projection whose K was split: added in
// order and rounded to bfloat16, as the kernel that adds partial sums would have stored them.
template <bool PARTIALS>
__global__ void rope_kv_write_bf16x8_kernel(bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ k, long k_stride,
                                            bf16_t* __restrict__ v, long v_stride, const int* __restrict__ positions,
                                            const int* __restrict__ seq_of_token, const float* __restrict__ inv_freq,
                                            bf16_t* __restrict__ cache, const int* __restrict__ block_table,
                                            int table_width, int page_size, int num_pages, int n_q_heads, int n_kv_heads,
                                            int head_dim, const float* __restrict__ partials, int n_partials,
                                            long partial_stride) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int pieces = head_dim / 8;
  const int piece = threadIdx.x;  // < pieces
  const int n_heads = n_q_heads + (k ? n_kv_heads : 0);
  bf16_t* kdst = nullptr;
  bf16_t* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }
  if (piece < pieces) {
    float c[4], s[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      c[e] = 1.f;
      s[e] = 0.f;
      if (inv_freq) sincosf((float)pos * inv_freq[4 * piece + e], &s[e], &c[e]);
    }
    // the blocks of a token (gridDim.y of them) take the heads in turn
    for (int hh = blockIdx.y * blockDim.y + threadIdx.y; hh < n_heads; hh += gridDim.y * blockDim.y) {
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      bf16_t* row = (is_key ? k + (size_t)t * k_stride : q + (size_t)t * q_stride) + (size_t)head * head_dim + 8 * piece;
      uint32_t w[4];
      if constexpr (PARTIALS) {
        const float* src = partials + (size_t)t * (n_q_heads + 2 * n_kv_heads) * head_dim + (size_t)hh * head_dim + 8 * piece;
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        for (int p = 0; p < n_partials; ++p) {
          const float4 a = *(const float4*)(src + (size_t)p * partial_stride);
          const float4 b = *(const float4*)(src + (size_t)p * partial_stride + 4);
          lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
          hi.x += b.x, hi.y += b.y, hi.z += b.z, hi.w += b.w;
        }
        w[0] = pack2_bf16(lo.x, lo.y), w[1] = pack2_bf16(lo.z, lo.w), w[2] = pack2_bf16(hi.x, hi.y), w[3] = pack2_bf16(hi.z, hi.w);
      } else {
        const uint4 in = *(const uint4*)row;
        w[0] = in.x, w[1] = in.y, w[2] = in.z, w[3] = in.w;
      }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float re = bf16_to_f32((bf16_t)(w[e] & 0xffffu));
        const float im = bf16_to_f32((bf16_t)(w[e] >> 16));
        o[e] = (uint32_t)f32_to_bf16(re * c[e] - im * s[e]) | ((uint32_t)f32_to_bf16(im * c[e] + re * s[e]) << 16);
      }
      const uint4 out = make_uint4(o[0], o[1], o[2], o[3]);
      if (inv_freq || PARTIALS) *(uint4*)row = out;
      if (is_key && kdst) *(uint4*)(kdst + ((size_t)head * page_size + slot) * head_dim + 8 * piece) = out;
    }
  }
  if ((vdst || PARTIALS) && v) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int tid = (blockIdx.y * blockDim.y + threadIdx.y) * blockDim.x + threadIdx.x;
    const int nthreads = gridDim.y * blockDim.x * blockDim.y;
    const int total = n_kv_heads * head_dim;
    bf16_t* vrow = v + (size_t)t * v_stride;
    for (int e = tid; e < total; e += nthreads) {
      const int head = e / head_dim;
      const int d = e - head * head_dim;
      bf16_t value;
      if constexpr (PARTIALS) {
        const float* src = partials + ((size_t)t * (n_q_heads + 2 * n_kv_heads) + n_q_heads + n_kv_heads) * head_dim + e;
        float sum = 0.f;
        for (int p = 0; p < n_partials; ++p) sum += src[(size_t)p * partial_stride];
        value = f32_to_bf16(sum);
        vrow[e] = value;
      } else {
        value = vrow[e];
      }
      if (vdst) vdst[(size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block] = value;
    }
  }
}

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ q, long q_stride, T* __restrict__ k, long k_stride,
                                     const T* __restrict__ v, long v_stride,
                                     const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                     const float* __restrict__ inv_freq, T* __restrict__ cache,
                                     const int* __restrict__ block_table, int table_width, int page_size,
                                     int num_pages, int n_q_heads, int n_kv_heads, int head_dim) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int i = threadIdx.x;  // pair index, < half
  const int n_heads = n_q_heads + (k ? n_kv_heads : 0);

  // where this token's key and value go
  T* kdst = nullptr;
  T* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }

  if (i < half) {
    float c = 1.f, s = 0.f;
    if (inv_freq) {
      const float a = (float)pos * inv_freq[i];
      sincosf(a, &s, &c);
    }
    for (int hh = threadIdx.y; hh < n_heads; hh += blockDim.y) {
      T* row;
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      if (is_key)
        row = k + (size_t)t * k_stride + (size_t)head * head_dim;
      else
        row = q + (size_t)t * q_stride + (size_t)head * head_dim;
      const float re = Elem<T>::load(row + 2 * i);
      const float im = Elem<T>::load(row + 2 * i + 1);
      const float ore = re * c - im * s;
      const float oim = im * c + re * s;
      if (inv_freq) {
        Elem<T>::store(row + 2 * i, ore);
        Elem<T>::store(row + 2 * i + 1, oim);
      }
      if (is_key && kdst) {
        T* dst = kdst + ((size_t)head * page_size + slot) * head_dim;
        Elem<T>::store(dst + 2 * i, ore);
        Elem<T>::store(dst + 2 * i + 1, oim);
      }
    }
  }

  if (vdst && v) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int tid = threadIdx.y * blockDim.x + threadIdx.x;
    const int nthreads = blockDim.x * blockDim.y;
    const int total = n_kv_heads * head_dim;
    const T* vrow = v + (size_t)t * v_stride;
    for (int e = tid; e < total; e += nthreads) {
      const int head = e / head_dim;
      const int d = e - head * head_dim;
      vdst[(size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block] = vrow[e];
    }
  }
}

extern "C" int cwm_rope_kv_write(void* q, long q_stride, void* k, long k_stride, const void* v, long v_stride,
                                 int dtype, const int* positions, const int* seq_of_token, const float* inv_freq,
                                 void* cache, const int* block_table, int table_width, int page_size,
                                 int num_pages, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                 hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0, "rope_kv_write: negative token count");
  CWM_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 1024,
              "rope_kv_write: head_dim %d must be even and at most 1024", head_dim);
  CWM_REQUIRE(n_q_heads >= 0 && n_kv_heads >= 0 && n_q_heads + n_kv_heads > 0, "rope_kv_write: no heads");
  CWM_REQUIRE(q || n_q_heads == 0, "rope_kv_write: queries missing");
  if (cache) {
    CWM_REQUIRE(k && v && block_table && seq_of_token, "rope_kv_write: a cache write needs k, v and a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0, "rope_kv_write: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  const int half = head_dim / 2;
  int bx = 1;
  while (bx < half) bx <<= 1;  // threads beyond `half` idle in the rotation
  int by = 256 / bx;
  if (by < 1) by = 1;
  const int heads = n_q_heads + n_kv_heads;
  if (by > heads) by = heads;
  dim3 block(bx, by);
  const bool rows16 = q_stride % 8 == 0 && k_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 &&
                      ((uintptr_t)cache % 16) == 0;
  if (dtype == CWM_BF16 && head_dim % 8 == 0 && head_dim <= 2048 && rows16) {
    int px = 1;
    while (px < head_dim / 8) px <<= 1;
    int py = 256 / px;
    if (py < 1) py = 1;
    if (py > heads) py = heads;
    // few tokens: several blocks a token, so that a decode step's rows are not left to as many blocks
    const int gy = n_tokens >= 1024 ? 1 : (heads + py - 1) / py;
    hipLaunchKernelGGL(rope_kv_write_bf16x8_kernel<false>, dim3(n_tokens, gy), dim3(px, py), 0, stream, (bf16_t*)q, q_stride,
                       (bf16_t*)k, k_stride, (bf16_t*)v, v_stride, positions, seq_of_token, inv_freq, (bf16_t*)cache,
                       block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads, head_dim, (const float*)nullptr, 0,
                       0L);
  } else if (dtype == CWM_F32)
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, dim3(n_tokens), block, 0, stream, (float*)q, q_stride,
                       (float*)k, k_stride, (const float*)v, v_stride, positions, seq_of_token, inv_freq,
                       (float*)cache, block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads,
                       head_dim);
  else if (dtype == CWM_BF16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, dim3(n_tokens), block, 0, stream, (bf16_t*)q, q_stride,
                       (bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, positions, seq_of_token, inv_freq,
                       (bf16_t*)cache, block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads,
                       head_dim);
  else
    return cwm_fail("rope_kv_write: unknown dtype %d", dtype);
  return cwm_launch_status("rope_kv_write");
}

// The same from the float32 partial sums [n_partials][n_tokens][(Hq + 2 Hkv) * head_dim] of the joined
// q/k/v projection (partial_stride elements apart): `qkv` [n_tokens][qkv_stride] receives the sums
// in bfloat16, q and k rotated, and the cache the rotated keys and the values.
extern "C" int cwm_rope_kv_write_partials(void* qkv, long qkv_stride, const float* partials, int n_partials,
                                          long partial_stride, const int* positions, const int* seq_of_token,
                                          const float* inv_freq, void* cache, const int* block_table, int table_width,
                                          int page_size, int num_pages, int n_tokens, int n_q_heads, int n_kv_heads,
                                          int head_dim, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_partials >= 1, "rope_kv_write_partials: bad sizes");
  CWM_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 2048, "rope_kv_write_partials: head_dim %d must be a multiple of 8", head_dim);
  CWM_REQUIRE(n_q_heads > 0 && n_kv_heads > 0, "rope_kv_write_partials: no heads");
  const long width = (long)(n_q_heads + 2 * n_kv_heads) * head_dim;
  CWM_REQUIRE(qkv && partials && positions, "rope_kv_write_partials: arguments missing");
  CWM_REQUIRE(qkv_stride >= width && qkv_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)partials % 16) == 0 &&
                  partial_stride % 4 == 0 && partial_stride >= (long)n_tokens * width,
              "rope_kv_write_partials: rows must be 16-byte aligned and the partial sums dense");
  if (cache) {
    CWM_REQUIRE(block_table && seq_of_token, "rope_kv_write_partials: a cache write needs a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0 && ((uintptr_t)cache % 16) == 0, "rope_kv_write_partials: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  int px = 1;
  while (px < head_dim / 8) px <<= 1;
  int py = 256 / px;
  if (py < 1) py = 1;
  if (py > n_q_heads + n_kv_heads) py = n_q_heads + n_kv_heads;
  bf16_t* q = (bf16_t*)qkv;
  bf16_t* k = q + (size_t)n_q_heads * head_dim;
  bf16_t* v = k + (size_t)n_kv_heads * head_dim;
  const int gy = n_tokens >= 1024 ? 1 : (n_q_heads + n_kv_heads + py - 1) / py;
  hipLaunchKernelGGL(rope_kv_write_bf16x8_kernel<true>, dim3(n_tokens, gy), dim3(px, py), 0, stream, q, qkv_stride, k, qkv_stride, v,
                     qkv_stride, positions, seq_of_token, inv_freq, (bf16_t*)cache, block_table, table_width, page_size,
                     num_pages, n_q_heads, n_kv_heads, head_dim, partials, n_partials, partial_stride);
  return cwm_launch_status("rope_kv_write_partials");
}

// ---- projection rows -> norm over the whole projection -> rotation -> cache ---------------------------- //
// A token's row of the joined projection is [q: Hq * qk_dim | k: Hkv * qk_dim | v: Hkv * v_dim] (type TS, or float32
// partial sums of a split K, added in order).  Queries and keys are each divided by the root mean square of the
// whole projection (all heads at once, eps inside the root) and multiplied by a weight per element, where a weight
// is given; then their heads are rotated by position * inv_freq[pair] (adjacent pairs; a frequency of 0 leaves its
// pair alone, so a table that ends in zeros rotates the leading dimensions only).  Heads are then laid out with
// `head_dim` elements, the common size of a cached key and value: a key's elements from qk_dim on and a value's
// from v_dim on are zeros (a zero adds nothing to a score, and the output columns it makes are dropped by the
// caller).  Queries go to q_out [T][Hq][head_dim], keys and values into the paged cache (layout at the top of
// this file).  All arithmetic float32; one block a token.
#define NORM_ROPE_MAX_HEAD 256

// four consecutive elements of a row, and of a cached key
template <typename T> struct Four;
template <> struct Four<float> {
  static __device__ __forceinline__ void add(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] += x.x, v[1] += x.y, v[2] += x.z, v[3] += x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Four<bf16_t> {
  static __device__ __forceinline__ void add(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *(const uint2*)p;
    v[0] += __uint_as_float(x.x << 16), v[1] += __uint_as_float(x.x & 0xffff0000u);
    v[2] += __uint_as_float(x.y << 16), v[3] += __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = pack2_bf16(v[0], v[1]);
    x.y = pack2_bf16(v[2], v[3]);
    *(uint2*)p = x;
  }
};

// The blocks of a token (gridDim.y of them) share its heads; each works out the token's two root mean squares itself.
// VEC: every size is a multiple of 4 and every row starts at a multiple of 16 bytes (8 for bfloat16): a thread
// takes four consecutive elements, two pairs, at a time.
template <typename TS, typename TO, bool VEC>
__global__ void __launch_bounds__(256)
qk_norm_rope_write_kernel(const TS* __restrict__ src, long src_stride, int n_partials, long partial_stride,
                          TO* __restrict__ q_out, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                          float eps, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                          const float* __restrict__ inv_freq, TO* __restrict__ cache, const int* __restrict__ block_table,
                          int table_width, int page_size, int num_pages, int n_q_heads, int n_kv_heads, int qk_dim,
                          int v_dim, int head_dim) {
  __shared__ float scratch[16];
  __shared__ __attribute__((aligned(16))) float cs[NORM_ROPE_MAX_HEAD];  // cos, sin of each pair
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int q_width = n_q_heads * qk_dim, k_width = n_kv_heads * qk_dim;
  const TS* srow = src + (size_t)t * src_stride;
  auto value = [&](int e) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += Elem<TS>::load(srow + (size_t)p * partial_stride + e);
    return v;
  };
  auto value4 = [&](int e, float (&v)[4]) {
    v[0] = v[1] = v[2] = v[3] = 0.f;
    for (int p = 0; p < n_partials; ++p) Four<TS>::add(srow + (size_t)p * partial_stride + e, v);
  };
  TO* kdst = nullptr;
  TO* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float c = 1.f, s = 0.f;
    const float f = inv_freq ? inv_freq[i] : 0.f;
    if (f != 0.f) sincosf((float)pos * f, &s, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = s;
  }
  float q_rstd = 1.f, k_rstd = 1.f;
  const bool norm_k = k_weight && cache;
  if (q_weight || norm_k) {
    // both sums of squares in one pass over [q | k]; each in the order of its own elements
    float sq = 0.f, sk = 0.f;
    const int first = q_weight ? 0 : q_width, last = norm_k ? q_width + k_width : q_width;
    if constexpr (VEC) {
      for (int e = first + 4 * threadIdx.x; e < last; e += 4 * blockDim.x) {
        float v[4];
        value4(e, v);
        const float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        if (e < q_width) sq += ss; else sk += ss;
      }
    } else {
      for (int e = first + threadIdx.x; e < last; e += blockDim.x) {
        const float v = value(e);
        if (e < q_width) sq += v * v; else sk += v * v;
      }
    }
    if (q_weight) q_rstd = 1.0f / sqrtf(block_sum(sq, scratch) / (float)q_width + eps);
    if (norm_k) k_rstd = 1.0f / sqrtf(block_sum(sk, scratch) / (float)k_width + eps);
  }
  __syncthreads();  // the table of cosines and sines is complete
  const int n_heads = n_q_heads + (cache ? n_kv_heads : 0);
  // this block's heads
  const int per_block = (n_heads + gridDim.y - 1) / gridDim.y;
  const int head_lo = blockIdx.y * per_block, head_hi = min(n_heads, head_lo + per_block);
  if constexpr (VEC) {
    const int quarter = head_dim / 4;
    for (int e = head_lo * quarter + threadIdx.x; e < head_hi * quarter; e += blockDim.x) {
      const int hh = e / quarter, d0 = 4 * (e - hh * quarter);
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (d0 < qk_dim) {
        value4((is_key ? q_width : 0) + head * qk_dim + d0, v);
        const float* weight = is_key ? k_weight : q_weight;
        if (weight) {
          const float rstd = is_key ? k_rstd : q_rstd;
          const float4 w = *(const float4*)(weight + head * qk_dim + d0);
          v[0] *= rstd * w.x, v[1] *= rstd * w.y, v[2] *= rstd * w.z, v[3] *= rstd * w.w;
        }
      }
      const float4 r = *(const float4*)(cs + d0);  // cos, sin of the pair d0 / 2 and of the next
      const float o[4] = {v[0] * r.x - v[1] * r.y, v[1] * r.x + v[0] * r.y, v[2] * r.z - v[3] * r.w, v[3] * r.z + v[2] * r.w};
      if (!is_key)
        Four<TO>::store(q_out + ((size_t)t * n_q_heads + head) * head_dim + d0, o);
      else if (kdst)
        Four<TO>::store(kdst + ((size_t)head * page_size + slot) * head_dim + d0, o);
    }
  } else {
    for (int e = head_lo * half + threadIdx.x; e < head_hi * half; e += blockDim.x) {
      const int hh = e / half, i = e - hh * half;
      const bool is_key = hh >= n_q_heads;
      const int head = is_key ? hh - n_q_heads : hh;
      const int base = (is_key ? q_width : 0) + head * qk_dim;
      const float* weight = is_key ? k_weight : q_weight;
      const float rstd = is_key ? k_rstd : q_rstd;
      float re = 0.f, im = 0.f;
      if (2 * i < qk_dim) re = value(base + 2 * i) * (weight ? rstd * weight[head * qk_dim + 2 * i] : 1.f);
      if (2 * i + 1 < qk_dim) im = value(base + 2 * i + 1) * (weight ? rstd * weight[head * qk_dim + 2 * i + 1] : 1.f);
      const float c = cs[2 * i], s = cs[2 * i + 1];
      const float ore = re * c - im * s, oim = im * c + re * s;
      TO* dst = nullptr;
      if (!is_key)
        dst = q_out + ((size_t)t * n_q_heads + head) * head_dim;
      else if (kdst)
        dst = kdst + ((size_t)head * page_size + slot) * head_dim;
      if (dst) {
        Elem<TO>::store(dst + 2 * i, ore);
        Elem<TO>::store(dst + 2 * i + 1, oim);
      }
    }
  }
  if (vdst) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int v_base = q_width + k_width;
    const int first = blockIdx.y * blockDim.x + threadIdx.x, step = gridDim.y * blockDim.x;
    if constexpr (VEC) {
      const int quarter = head_dim / 4;
      for (int e = first; e < n_kv_heads * quarter; e += step) {
        const int head = e / quarter, d0 = 4 * (e - head * quarter);
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (d0 < v_dim) value4(v_base + head * v_dim + d0, v);
        TO* dst = vdst + (size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d0) * v_block + slot % v_block;
#pragma unroll
        for (int i = 0; i < 4; ++i) Elem<TO>::store(dst + (size_t)i * v_block, v[i]);
      }
    } else {
      for (int e = first; e < n_kv_heads * head_dim; e += step) {
        const int head = e / head_dim, d = e - head * head_dim;
        const float v = d < v_dim ? value(v_base + head * v_dim + d) : 0.f;
        Elem<TO>::store(vdst + (size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block, v);
      }
    }
  }
}

// src: [n_tokens][src_stride] of src_dtype, or n_partials float32 slabs partial_stride apart.  q_weight [Hq * qk_dim],
// k_weight [Hkv * qk_dim]: float32, null for no norm.  inv_freq: float32 [head_dim / 2] or null.  cache: null where
// only the queries are wanted (a layer that reads a cache written by another).
extern "C" int cwm_qk_norm_rope_write(const void* src, int src_dtype, long src_stride, int n_partials, long partial_stride,
                                      void* q_out, int out_dtype, const float* q_weight, const float* k_weight, float eps,
                                      const int* positions, const int* seq_of_token, const float* inv_freq, void* cache,
                                      const int* block_table, int table_width, int page_size, int num_pages, int n_tokens,
                                      int n_q_heads, int n_kv_heads, int qk_dim, int v_dim, int head_dim, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_partials >= 1, "qk_norm_rope_write: bad sizes");
  CWM_REQUIRE(n_partials == 1 || src_dtype == CWM_F32, "qk_norm_rope_write: partial sums must be float32");
  CWM_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= NORM_ROPE_MAX_HEAD,
              "qk_norm_rope_write: head_dim %d must be even and at most %d", head_dim, NORM_ROPE_MAX_HEAD);
  CWM_REQUIRE(qk_dim >= 1 && v_dim >= 1 && qk_dim <= head_dim && v_dim <= head_dim,
              "qk_norm_rope_write: heads of %d (queries, keys) and %d (values) do not fit the cached head of %d", qk_dim, v_dim, head_dim);
  CWM_REQUIRE(n_q_heads > 0 && (n_kv_heads > 0 || (n_kv_heads == 0 && !cache)), "qk_norm_rope_write: no heads");
  CWM_REQUIRE(src && q_out && positions, "qk_norm_rope_write: arguments missing");
  CWM_REQUIRE(eps > 0.f || (!q_weight && !k_weight), "qk_norm_rope_write: eps must be positive");
  if (cache) {
    CWM_REQUIRE(block_table && seq_of_token, "qk_norm_rope_write: a cache write needs a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0, "qk_norm_rope_write: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  const int key = (src_dtype << 1) | out_dtype;
  const int src_bytes = src_dtype == CWM_F32 ? 4 : 2, out_bytes = out_dtype == CWM_F32 ? 4 : 2;
  const bool vec = qk_dim % 4 == 0 && v_dim % 4 == 0 && head_dim % 4 == 0 && src_stride % 4 == 0 && partial_stride % 4 == 0 &&
                   ((uintptr_t)src % (4 * src_bytes)) == 0 && ((uintptr_t)q_out % (4 * out_bytes)) == 0 &&
                   ((uintptr_t)cache % (4 * out_bytes)) == 0 && ((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0;
  // few tokens: several blocks a token, so that a decode step's rows are not left to as many blocks
  const int heads = n_q_heads + n_kv_heads;
  const int gy = n_tokens >= 512 ? 1 : (heads < 8 ? heads : 8);
#define CWM_NORM_ROPE_V(TS, TO, VEC)                                                                                       \
  hipLaunchKernelGGL((qk_norm_rope_write_kernel<TS, TO, VEC>), dim3(n_tokens, gy), dim3(256), 0, stream, (const TS*)src,    \
                     src_stride, n_partials, partial_stride, (TO*)q_out, q_weight, k_weight, eps, positions, seq_of_token, \
                     inv_freq, (TO*)cache, block_table, table_width, page_size, num_pages, n_q_heads, n_kv_heads, qk_dim,  \
                     v_dim, head_dim)
#define CWM_NORM_ROPE(TS, TO)          \
  do {                                 \
    if (vec)                           \
      CWM_NORM_ROPE_V(TS, TO, true);   \
    else                               \
      CWM_NORM_ROPE_V(TS, TO, false);  \
  } while (0)
  switch (key) {
    case 0: CWM_NORM_ROPE(float, float); break;
    case 1: CWM_NORM_ROPE(float, bf16_t); break;
    case 3: CWM_NORM_ROPE(bf16_t, bf16_t); break;
    default: return cwm_fail("qk_norm_rope_write: source type %d with cache type %d is not built", src_dtype, out_dtype);
  }
#undef CWM_NORM_ROPE
#undef CWM_NORM_ROPE_V
  return cwm_launch_status("qk_norm_rope_write");
}

// ---- projection rows -> bias -> norm of every head -> rotation -> (values mixed with another layer's) -> cache -- //
// A token's row of the joined projection is [q: Hq * qk_dim | k: Hkv * qk_dim | v: Hkv * v_dim | ...] (type TS, or
// float32 partial sums of a split K, added in order), to which `bias` (float32, one value a column of q, k and v) is
// added.  Every query head and every key head is divided by its own root mean square (eps inside the root) and
// multiplied by a weight of qk_dim values that all heads share, where a weight is given; then rotated by
// position * inv_freq[pair] (adjacent pairs; a frequency of 0 leaves its pair alone).  Values: where `v_other` is
// given, v <- (1 - mix) v + mix v_other, with `mix` one float32 on the device and v_other [T][Hkv * v_dim] the
// values that another layer made of the same tokens; `v_keep`, where given, receives this layer's values as they go
// into the cache, [T][Hkv * v_dim].  Heads are laid out with `head_dim` elements as in the kernel above.  All
// arithmetic float32.  A wavefront a head: the lanes hold the head's pairs, so a head's sum of squares is one
// reduction over the lanes; the blocks of a token (gridDim.y of them) share its heads.
template <typename TS, typename TO>
__global__ void __launch_bounds__(256)
head_norm_rope_write_kernel(const TS* __restrict__ src, long src_stride, int n_partials, long partial_stride,
                            const float* __restrict__ bias, TO* __restrict__ q_out, const float* __restrict__ q_weight,
                            const float* __restrict__ k_weight, float eps, const int* __restrict__ positions,
                            const int* __restrict__ seq_of_token, const float* __restrict__ inv_freq, TO* __restrict__ cache,
                            const int* __restrict__ block_table, int table_width, int page_size, int num_pages, int n_q_heads,
                            int n_kv_heads, int qk_dim, int v_dim, int head_dim, const TO* __restrict__ v_other,
                            long v_other_stride, const float* __restrict__ v_mix, TO* __restrict__ v_keep) {
  __shared__ __attribute__((aligned(16))) float cs[NORM_ROPE_MAX_HEAD];  // cos, sin of each pair
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const int wave = threadIdx.x / CWM_WAVE;
  const int q_width = n_q_heads * qk_dim, k_width = n_kv_heads * qk_dim;
  const TS* srow = src + (size_t)t * src_stride;
  auto value = [&](int e) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += Elem<TS>::load(srow + (size_t)p * partial_stride + e);
    return bias ? v + bias[e] : v;
  };
  TO* kdst = nullptr;
  TO* vdst = nullptr;
  int slot = 0;
  if (cache) {
    const int seq = seq_of_token[t];
    const int lp = pos / page_size;
    slot = pos - lp * page_size;
    const int page = (lp >= 0 && lp < table_width) ? block_table[(size_t)seq * table_width + lp] : -1;
    if (page >= 0 && page < num_pages) {
      const size_t plane = (size_t)n_kv_heads * page_size * head_dim;
      kdst = cache + (size_t)page * 2 * plane;
      vdst = kdst + plane;
    }
  }
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float c = 1.f, s = 0.f;
    const float f = inv_freq ? inv_freq[i] : 0.f;
    if (f != 0.f) sincosf((float)pos * f, &s, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = s;
  }
  __syncthreads();
  const int n_heads = n_q_heads + (cache ? n_kv_heads : 0);
  const int waves = blockDim.x / CWM_WAVE;
  for (int hh = blockIdx.y * waves + wave; hh < n_heads; hh += gridDim.y * waves) {
    const bool is_key = hh >= n_q_heads;
    const int head = is_key ? hh - n_q_heads : hh;
    const int base = (is_key ? q_width : 0) + head * qk_dim;
    const float* weight = is_key ? k_weight : q_weight;
    // pairs lane, lane + 64 of the head
    float re[2], im[2];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int i = lane + CWM_WAVE * r;
      re[r] = (i < half && 2 * i < qk_dim) ? value(base + 2 * i) : 0.f;
      im[r] = (i < half && 2 * i + 1 < qk_dim) ? value(base + 2 * i + 1) : 0.f;
      ss += re[r] * re[r] + im[r] * im[r];
    }
    float rstd = 1.f;
    if (weight) rstd = 1.0f / sqrtf(wave_sum(ss) / (float)qk_dim + eps);
    TO* dst = nullptr;
    if (!is_key)
      dst = q_out + ((size_t)t * n_q_heads + head) * head_dim;
    else if (kdst)
      dst = kdst + ((size_t)head * page_size + slot) * head_dim;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int i = lane + CWM_WAVE * r;
      if (i < half && dst) {
        float a = re[r], b = im[r];
        if (weight) {
          a *= rstd * (2 * i < qk_dim ? weight[2 * i] : 0.f);
          b *= rstd * (2 * i + 1 < qk_dim ? weight[2 * i + 1] : 0.f);
        }
        const float c = cs[2 * i], s = cs[2 * i + 1];
        Elem<TO>::store(dst + 2 * i, a * c - b * s);
        Elem<TO>::store(dst + 2 * i + 1, b * c + a * s);
      }
    }
  }
  if (vdst || v_keep) {
    const int v_block = (page_size % 8 == 0) ? 8 : page_size;
    const int v_base = q_width + k_width;
    const float mix = (v_other && v_mix) ? *v_mix : 0.f;
    for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < n_kv_heads * head_dim; e += gridDim.y * blockDim.x) {
      const int head = e / head_dim, d = e - head * head_dim;
      float v = 0.f;
      if (d < v_dim) {
        v = value(v_base + head * v_dim + d);
        if (v_other) v = (1.0f - mix) * v + mix * Elem<TO>::load(v_other + (size_t)t * v_other_stride + head * v_dim + d);
        if (v_keep) Elem<TO>::store(v_keep + ((size_t)t * n_kv_heads + head) * v_dim + d, v);
      }
      if (vdst)
        Elem<TO>::store(vdst + (size_t)head * head_dim * page_size + ((size_t)(slot / v_block) * head_dim + d) * v_block + slot % v_block, v);
    }
  }
}

// src: [n_tokens][src_stride] of src_dtype (the row may go on beyond q, k and v), or n_partials float32 slabs
// partial_stride apart.  bias: float32 [(Hq + Hkv) * qk_dim + Hkv * v_dim] or null.  q_weight, k_weight: float32
// [qk_dim] or null.  inv_freq: float32 [head_dim / 2] or null.  v_other ([n_tokens][v_other_stride], the cache's type)
// with v_mix (one float32 on the device): both or neither.  v_keep: [n_tokens][Hkv * v_dim] of the cache's type, or null.
extern "C" int cwm_head_norm_rope_write(const void* src, int src_dtype, long src_stride, int n_partials, long partial_stride,
                                        const float* bias, void* q_out, int out_dtype, const float* q_weight, const float* k_weight,
                                        float eps, const int* positions, const int* seq_of_token, const float* inv_freq, void* cache,
                                        const int* block_table, int table_width, int page_size, int num_pages, int n_tokens,
                                        int n_q_heads, int n_kv_heads, int qk_dim, int v_dim, int head_dim, const void* v_other,
                                        long v_other_stride, const float* v_mix, void* v_keep, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_partials >= 1, "head_norm_rope_write: bad sizes");
  CWM_REQUIRE(n_partials == 1 || src_dtype == CWM_F32, "head_norm_rope_write: partial sums must be float32");
  CWM_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= NORM_ROPE_MAX_HEAD,
              "head_norm_rope_write: head_dim %d must be even and at most %d", head_dim, NORM_ROPE_MAX_HEAD);
  CWM_REQUIRE(qk_dim >= 1 && v_dim >= 1 && qk_dim <= head_dim && v_dim <= head_dim,
              "head_norm_rope_write: heads of %d (queries, keys) and %d (values) do not fit the cached head of %d", qk_dim, v_dim, head_dim);
  CWM_REQUIRE(n_q_heads > 0 && n_kv_heads > 0, "head_norm_rope_write: no heads");
  CWM_REQUIRE(src && q_out && positions, "head_norm_rope_write: arguments missing");
  CWM_REQUIRE(eps > 0.f || (!q_weight && !k_weight), "head_norm_rope_write: eps must be positive");
  CWM_REQUIRE((v_other == nullptr) == (v_mix == nullptr), "head_norm_rope_write: other values and their weight come together");
  if (cache) {
    CWM_REQUIRE(block_table && seq_of_token, "head_norm_rope_write: a cache write needs a block table");
    CWM_REQUIRE(page_size > 0 && num_pages > 0 && table_width > 0, "head_norm_rope_write: bad cache geometry");
  }
  if (n_tokens == 0) return 0;
  const int key = (src_dtype << 1) | out_dtype;
  // few tokens: several blocks a token, so that a decode step's rows are not left to as many blocks
  const int heads = n_q_heads + n_kv_heads;
  const int gy = n_tokens >= 512 ? 1 : (heads <= 4 ? 1 : (heads < 32 ? (heads + 3) / 4 : 8));
#define CWM_HEAD_NORM_ROPE(TS, TO)                                                                                         \
  hipLaunchKernelGGL((head_norm_rope_write_kernel<TS, TO>), dim3(n_tokens, gy), dim3(256), 0, stream, (const TS*)src,       \
                     src_stride, n_partials, partial_stride, bias, (TO*)q_out, q_weight, k_weight, eps, positions,         \
                     seq_of_token, inv_freq, (TO*)cache, block_table, table_width, page_size, num_pages, n_q_heads,        \
                     n_kv_heads, qk_dim, v_dim, head_dim, (const TO*)v_other, v_other_stride, v_mix, (TO*)v_keep)
  switch (key) {
    case 0: CWM_HEAD_NORM_ROPE(float, float); break;
    case 1: CWM_HEAD_NORM_ROPE(float, bf16_t); break;
    case 3: CWM_HEAD_NORM_ROPE(bf16_t, bf16_t); break;
    default: return cwm_fail("head_norm_rope_write: source type %d with cache type %d is not built", src_dtype, out_dtype);
  }
#undef CWM_HEAD_NORM_ROPE
  return cwm_launch_status("head_norm_rope_write");
}
