// A matrix memory with exponential gates and a running maximum (the mLSTM recurrence), with a per-request state.
//
// Per head, with S (d x e), n (d) and a maximum m, all zero when a request starts (m too: zero, not minus infinity):
//     i_t = c tanh(a_t / c),   f_t = logsigmoid(c tanh(b_t / c))        a_t, b_t: the two gate projections, c the cap
//     m_t = max(f_t + m_(t-1), i_t)
//     S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,      n_t the same with k_t alone
//     y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),                 q_t already scaled
// Everything but the loads of q, k and v is float32, and tokens are walked one by one in order, so a portion of a
// prompt gives the same bits as the same tokens one at a time.
//
// Two kernels.  `memory_gates_kernel` (a wavefront a (head, sequence)) walks the gates, the maximum and n, which
// need d values a token, and leaves three numbers a token: the factor of the old state, the factor of k v^T and
// the denominator.  `memory_scan_kernel` (a block a (tile of value columns, head, sequence)) walks S with those: a
// thread holds 16 rows of one column, `split` lanes share a column and add their parts of S^T q by shuffles, and q,
// k, v and the three numbers of 16 tokens are staged through LDS.  `memory_out_kernel` then divides every head's y by
// its root mean square, multiplies by a weight and by sigmoid(gate).
//
// State of a request, float32: per head [e][d_pad] (S transposed: a column's rows side by side, d_pad = 16 * split),
// then n [d_pad], then m and three unused values.
#include "common.h"

CWM_DEFINE_ERROR_API

#define MEM_ROWS 16        // rows of a column that one thread holds
#define MEM_MAX_DIM 256    // largest d: 16 lanes a column
#define MEM_CHUNK 16       // tokens staged at once
#define MEM_THREADS 256

extern "C" int cwm_matrix_memory_max_dim() { return MEM_MAX_DIM; }

// lanes that share a column: the least power of two with 16 * split >= d
static inline int mem_split(int d) {
  int s = 1;
  while (MEM_ROWS * s < d) s *= 2;
  return s;
}

extern "C" int cwm_matrix_memory_split(int d) { return mem_split(d); }

// elements of one head's state, and of a request's
extern "C" long cwm_matrix_memory_head_elems(int d, int e) {
  const long d_pad = MEM_ROWS * mem_split(d);
  return (long)e * d_pad + d_pad + 4;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// coef: float32 [T][heads][4]: {factor of the old state, factor of k v^T, denominator, unused}
template <typename T>
__global__ void __launch_bounds__(CWM_WAVE)
memory_gates_kernel(const T* __restrict__ src, long src_stride, int q_off, int k_off, const float* __restrict__ gates,
                    long gates_stride, float cap, float q_scale, float* __restrict__ state, long state_stride, long head_elems,
                    const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ coef, int heads,
                    int d, int e, int d_pad) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  float* st = state + (size_t)state_slots[b] * state_stride + (size_t)h * head_elems + (size_t)e * d_pad;
  float n[MEM_MAX_DIM / CWM_WAVE];
#pragma unroll
  for (int r = 0; r < MEM_MAX_DIM / CWM_WAVE; ++r) {
    const int row = lane + CWM_WAVE * r;
    n[r] = row < d ? st[row] : 0.f;
  }
  float m = st[d_pad];
  const float inv_cap = 1.0f / cap;
  for (int base = t0; base < t1; base += CWM_WAVE) {
    // the gates of 64 tokens, a lane a token
    float gi = 0.f, gf = 0.f;
    if (base + lane < t1) {
      const float* g = gates + (size_t)(base + lane) * gates_stride;
      gi = cap * tanhf(g[h] * inv_cap);
      gf = log_sigmoid(cap * tanhf(g[heads + h] * inv_cap));
    }
    const int count = min(CWM_WAVE, t1 - base);
    float kk[MEM_MAX_DIM / CWM_WAVE], qq[MEM_MAX_DIM / CWM_WAVE];
    auto fetch = [&](int t) {
      const T* row = src + (size_t)t * src_stride + (size_t)h * d;
#pragma unroll
      for (int r = 0; r < MEM_MAX_DIM / CWM_WAVE; ++r) {
        const int x = lane + CWM_WAVE * r;
        kk[r] = x < d ? Elem<T>::load(row + k_off + x) : 0.f;
        qq[r] = x < d ? Elem<T>::load(row + q_off + x) * q_scale : 0.f;
      }
    };
    fetch(base);
    for (int j = 0; j < count; ++j) {
      const float i_t = __shfl(gi, j, CWM_WAVE), f_t = __shfl(gf, j, CWM_WAVE);
      const float m_new = fmaxf(f_t + m, i_t);
      const float keep = expf(f_t + m - m_new), take = expf(i_t - m_new);
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < MEM_MAX_DIM / CWM_WAVE; ++r) {
        n[r] = fmaf(keep, n[r], take * kk[r]);
        dot = fmaf(n[r], qq[r], dot);
      }
      if (j + 1 < count) fetch(base + j + 1);  // on its way during the reduction
      dot = wave_sum(dot);
      m = m_new;
      if (lane == 0) {
        float* c = coef + ((size_t)(base + j) * heads + h) * 4;
        *(float4*)c = make_float4(keep, take, fmaxf(fabsf(dot), expf(-m_new)) + 1e-6f, 0.f);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < MEM_MAX_DIM / CWM_WAVE; ++r) {
    const int row = lane + CWM_WAVE * r;
    if (row < d) st[row] = n[r];
  }
  if (lane == 0) st[d_pad] = m;
}

// y: float32 [T][heads * e]
template <typename T>
__global__ void __launch_bounds__(MEM_THREADS)
memory_scan_kernel(const T* __restrict__ src, long src_stride, int q_off, int k_off, int v_off, float q_scale,
                   const float* __restrict__ coef, float* __restrict__ state, long state_stride, long head_elems,
                   const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ y, int heads, int d,
                   int e, int split) {
  __shared__ __attribute__((aligned(16))) float q_s[MEM_CHUNK][MEM_MAX_DIM];
  __shared__ __attribute__((aligned(16))) float k_s[MEM_CHUNK][MEM_MAX_DIM];
  __shared__ float v_s[MEM_CHUNK][MEM_THREADS];  // a token's values; its results take their place once they are used
  __shared__ __attribute__((aligned(16))) float c_s[MEM_CHUNK][4];
  const int h = blockIdx.y, b = blockIdx.z;
  const int d_pad = MEM_ROWS * split;
  const int cols = MEM_THREADS / split;  // value columns of a block
  const int c_local = threadIdx.x / split, s = threadIdx.x - c_local * split;
  const int col = blockIdx.x * cols + c_local;
  const bool live = col < e;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  float* st = state + (size_t)state_slots[b] * state_stride + (size_t)h * head_elems + (size_t)col * d_pad;
  // rows 4 (s + split j) .. + 3, j = 0..3: the lanes of a column read 16 bytes each of consecutive memory
  float S[MEM_ROWS];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) x = *(const float4*)(st + 4 * (s + split * j));
    S[4 * j] = x.x, S[4 * j + 1] = x.y, S[4 * j + 2] = x.z, S[4 * j + 3] = x.w;
  }
  for (int base = t0; base < t1; base += MEM_CHUNK) {
    const int count = min(MEM_CHUNK, t1 - base);
    __syncthreads();  // the chunk before has been walked and its results stored
    for (int x = threadIdx.x; x < count * d_pad; x += MEM_THREADS) {
      const int tok = x / d_pad, r = x - tok * d_pad;
      const T* row = src + (size_t)(base + tok) * src_stride + (size_t)h * d;
      q_s[tok][r] = r < d ? Elem<T>::load(row + q_off + r) * q_scale : 0.f;
      k_s[tok][r] = r < d ? Elem<T>::load(row + k_off + r) : 0.f;
    }
    for (int x = threadIdx.x; x < count * cols; x += MEM_THREADS) {
      const int tok = x / cols, c = x - tok * cols;
      const int cc = blockIdx.x * cols + c;
      v_s[tok][c] = cc < e ? Elem<T>::load(src + (size_t)(base + tok) * src_stride + v_off + (size_t)h * e + cc) : 0.f;
    }
    if (threadIdx.x < count) *(float4*)c_s[threadIdx.x] = *(const float4*)(coef + ((size_t)(base + threadIdx.x) * heads + h) * 4);
    __syncthreads();
    for (int tok = 0; tok < count; ++tok) {
      const float4 c = *(const float4*)c_s[tok];
      const float tv = c.y * v_s[tok][c_local];
      float num = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 kk = *(const float4*)(&k_s[tok][4 * (s + split * j)]);
        const float4 qq = *(const float4*)(&q_s[tok][4 * (s + split * j)]);
        S[4 * j] = fmaf(c.x, S[4 * j], kk.x * tv);
        S[4 * j + 1] = fmaf(c.x, S[4 * j + 1], kk.y * tv);
        S[4 * j + 2] = fmaf(c.x, S[4 * j + 2], kk.z * tv);
        S[4 * j + 3] = fmaf(c.x, S[4 * j + 3], kk.w * tv);
        num = fmaf(S[4 * j], qq.x, num);
        num = fmaf(S[4 * j + 1], qq.y, num);
        num = fmaf(S[4 * j + 2], qq.z, num);
        num = fmaf(S[4 * j + 3], qq.w, num);
      }
      for (int off = 1; off < split; off <<= 1) num += __shfl_xor(num, off, CWM_WAVE);
      if (s == 0) v_s[tok][c_local] = num / c.z;  // the column's lanes, all in this wavefront, have read the value
    }
    __syncthreads();
    for (int x = threadIdx.x; x < count * cols; x += MEM_THREADS) {
      const int tok = x / cols, c = x - tok * cols;
      const int cc = blockIdx.x * cols + c;
      if (cc < e) y[(size_t)(base + tok) * heads * e + (size_t)h * e + cc] = v_s[tok][c];
    }
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < 4; ++j) *(float4*)(st + 4 * (s + split * j)) = make_float4(S[4 * j], S[4 * j + 1], S[4 * j + 2], S[4 * j + 3]);
  }
}

// out[t][h * e + c] = y[t][h * e + c] / sqrt(mean_c(y[t][h]^2) + eps) * weight[h * e + c] * sigmoid(gate[t][h * e + c]);
// a wavefront a (token, head)
template <typename T>
__global__ void __launch_bounds__(MEM_THREADS)
memory_out_kernel(const float* __restrict__ y, const float* __restrict__ weight, const T* __restrict__ gate, long gate_stride,
                  T* __restrict__ out, long n_pairs, int heads, int e, float eps) {
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const long pair = (long)blockIdx.x * (MEM_THREADS / CWM_WAVE) + threadIdx.x / CWM_WAVE;
  if (pair >= n_pairs) return;
  const long t = pair / heads;
  const int h = (int)(pair - t * heads);
  const float* row = y + (size_t)t * heads * e + (size_t)h * e;
  float ss = 0.f;
  for (int c = lane; c < e; c += CWM_WAVE) ss = fmaf(row[c], row[c], ss);
  const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)e + eps);
  for (int c = lane; c < e; c += CWM_WAVE) {
    const float g = Elem<T>::load(gate + (size_t)t * gate_stride + (size_t)h * e + c);
    Elem<T>::store(out + (size_t)t * heads * e + (size_t)h * e + c, row[c] * rstd * weight[h * e + c] / (1.0f + expf(-g)));
  }
}

// src: the joined projection [n_tokens][src_stride] of dtype: q at column q_off (heads * d), k at k_off (heads * d), v at
// v_off (heads * e), the output gate at g_off (heads * e).  gates: float32 [n_tokens][gates_stride], the input gates'
// projection in columns 0..heads-1 and the forget gates' in heads..2 heads-1, biases included.  state: float32
// [slots][state_stride].  coef: float32 scratch [n_tokens][heads][4]; y: float32 scratch [n_tokens][heads * e].
// out: [n_tokens][heads * e] of dtype.
extern "C" int cwm_matrix_memory(const void* src, int dtype, long src_stride, int q_off, int k_off, int v_off, int g_off,
                                 const float* gates, long gates_stride, float cap, float q_scale, float* state, long state_stride,
                                 int n_slots, const int* cu_q, const int* state_slots, int n_seqs, int n_tokens,
                                 float* coef, float* y, const float* weight, float eps, void* out, int heads, int d, int e,
                                 hipStream_t stream) {
  CWM_REQUIRE(heads >= 1 && d >= 1 && e >= 1 && d <= MEM_MAX_DIM, "matrix_memory: heads of %d x %d: d must lie in 1..%d", d, e, MEM_MAX_DIM);
  CWM_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && n_slots >= 1, "matrix_memory: bad counts");
  CWM_REQUIRE(cap > 0.f && eps > 0.f, "matrix_memory: the gates' cap and eps must be positive");
  const int split = mem_split(d);
  const long head_elems = cwm_matrix_memory_head_elems(d, e);
  CWM_REQUIRE(state_stride >= heads * head_elems && state_stride % 4 == 0 && ((uintptr_t)state % 16) == 0,
              "matrix_memory: a request's state needs %ld values, 16-byte aligned", heads * head_elems);
  CWM_REQUIRE(src && gates && state && cu_q && state_slots && coef && y && weight && out, "matrix_memory: arguments missing");
  CWM_REQUIRE(((uintptr_t)coef % 16) == 0, "matrix_memory: scratch must be 16-byte aligned");
  if (n_seqs == 0 || n_tokens == 0) return 0;
  CWM_REQUIRE(n_seqs <= 65535, "matrix_memory: too many sequences for one launch");
  const int cols = MEM_THREADS / split;
  const int tiles = (e + cols - 1) / cols;
  const long n_pairs = (long)n_tokens * heads;
  const unsigned out_blocks = (unsigned)((n_pairs + MEM_THREADS / CWM_WAVE - 1) / (MEM_THREADS / CWM_WAVE));
#define CWM_MEMORY(T)                                                                                                       \
  do {                                                                                                                      \
    hipLaunchKernelGGL(memory_gates_kernel<T>, dim3(heads, n_seqs), dim3(CWM_WAVE), 0, stream, (const T*)src, src_stride,    \
                       q_off, k_off, gates, gates_stride, cap, q_scale, state, state_stride, head_elems, cu_q, state_slots, \
                       coef, heads, d, e, MEM_ROWS * split);                                                                \
    hipLaunchKernelGGL(memory_scan_kernel<T>, dim3(tiles, heads, n_seqs), dim3(MEM_THREADS), 0, stream, (const T*)src,       \
                       src_stride, q_off, k_off, v_off, q_scale, (const float*)coef, state, state_stride, head_elems, cu_q, \
                       state_slots, y, heads, d, e, split);                                                                 \
    hipLaunchKernelGGL(memory_out_kernel<T>, dim3(out_blocks), dim3(MEM_THREADS), 0, stream, (const float*)y, weight,        \
                       (const T*)src + g_off, src_stride, (T*)out, n_pairs, heads, e, eps);                                 \
  } while (0)
  if (dtype == CWM_F32)
    CWM_MEMORY(float);
  else if (dtype == CWM_BF16)
    CWM_MEMORY(bf16_t);
  else
    return cwm_fail("matrix_memory: unknown type %d", dtype);
#undef CWM_MEMORY
  return cwm_launch_status("matrix_memory");
}
