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
// Short portions (decoding among them) are walked by two kernels.  `memory_gates_kernel` (a wavefront a (head, sequence)) walks the gates, the maximum and n, which
// need d values a token, and leaves three numbers a token: the factor of the old state, the factor of k v^T and
// the denominator.  `memory_scan_kernel` (a block a (tile of value columns, head, sequence)) walks S with those: a
// thread holds 16 rows of one column, `split` lanes share a column and add their parts of S^T q by shuffles, and q,
// k, v and the three numbers of 16 tokens are staged through LDS.  `memory_out_kernel` then divides every head's y by
// its root mean square, multiplies by a weight and by sigmoid(gate).
//
// A step with a long portion takes blocks of MEMC_L tokens at once instead.  With b_t the sum of f up to t, a_s = i_s - b_s
// and g_t = m_t - b_t, the recurrence unrolls to
//     S_t = exp(g_c - g_t) S_c + sum_(c < s <= t) exp(a_s - g_t) k_s v_s^T        (c: the token before the block)
// with no exponent above zero, so a block's results are (Q K^T, weighted and masked) V + (weighted Q) S_c, and the state
// moves once a block.  `memory_maxima_kernel` walks m (a thread block a (head, sequence), the same float32 operations as the
// walk above, so both give the same m) and sums f in float64, since differences of long sums are taken;
// `memory_scores_kernel` works out every block's weighted scores and weights side by side, and `memory_chunk_kernel` (a thread
// block a (tile of value columns, head, sequence)) walks the blocks with the remaining products on the float32 matrix
// instruction.  The normaliser n
// is the column after the last value column, with ones for values, so n_t . q_t falls out as that column's result and the
// division moves into `memory_out_kernel`.  This differs from the walk by rounding only.
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

#define MEMC_L 32         // tokens of a block
#define MEMC_COLS 32      // value columns of a thread block
#define MEMC_THREADS 512
#define MEMC_GROUPS (MEMC_THREADS / MEMC_COLS)  // groups of rows
#define MEMC_WAVES (MEMC_THREADS / CWM_WAVE)
#define MEMX_THREADS 256
static_assert(MEMC_COLS == MEMC_L, "a block's scores are staged like its values");
#define MEMX_SPAN 1024    // tokens whose gates are worked out side by side before the maximum walks them

// coef: float32 [T][heads][4]: {i_t, m_t, b_t as a float64 in two words}; b counts from the portion's start.
// start: float64 [n_seqs][heads]: m before the portion.
__global__ void __launch_bounds__(MEMX_THREADS)
memory_maxima_kernel(const float* __restrict__ gates, long gates_stride, float cap, float* __restrict__ state, long state_stride,
                     long head_elems, const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ coef,
                     double* __restrict__ start, int heads, int e, int d_pad) {
  __shared__ float gi_s[MEMX_SPAN], gf_s[MEMX_SPAN];
  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const bool walker = threadIdx.x < CWM_WAVE;  // the first wavefront walks; all work out gates
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  float* st_m = state + (size_t)state_slots[b] * state_stride + (size_t)h * head_elems + (size_t)e * d_pad + d_pad;
  float m = *st_m;
  if (threadIdx.x == 0) start[(size_t)b * heads + h] = (double)m;
  const float inv_cap = 1.0f / cap;
  double before = 0.0;
  for (int span = t0; span < t1; span += MEMX_SPAN) {
    const int n = min(MEMX_SPAN, t1 - span);
    __syncthreads();  // the span before has been walked
    for (int x = threadIdx.x; x < n; x += MEMX_THREADS) {
      const float* g = gates + (size_t)(span + x) * gates_stride;
      gi_s[x] = cap * tanhf(g[h] * inv_cap);
      gf_s[x] = log_sigmoid(cap * tanhf(g[heads + h] * inv_cap));
    }
    __syncthreads();
    if (!walker) continue;
    for (int base = 0; base < n; base += CWM_WAVE) {
      const int count = min(CWM_WAVE, n - base);
      // beyond the portion's end: gates that leave m as it is, so the walk below needs no branch
      const float gi = lane < count ? gi_s[base + lane] : -INFINITY, gf = lane < count ? gf_s[base + lane] : 0.f;
      double sum = (double)gf;  // zero beyond the portion's end
#pragma unroll
      for (int off = 1; off < CWM_WAVE; off <<= 1) {
        const double o = __shfl_up(sum, off, CWM_WAVE);
        if (lane >= off) sum += o;
      }
      float mine = 0.f;
#pragma unroll
      for (int j = 0; j < CWM_WAVE; ++j) {
        // (a lane known when compiling: read through a scalar register, not through LDS)
        const float fj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gf), j));
        const float ij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gi), j));
        m = fmaxf(fj + m, ij);
        mine = lane == j ? m : mine;
      }
      if (lane < count) {
        float* c = coef + ((size_t)(span + base + lane) * heads + h) * 4;
        c[0] = gi, c[1] = mine;
        *(double*)(c + 2) = before + sum;
      }
      before += __shfl(sum, CWM_WAVE - 1, CWM_WAVE);
    }
  }
  if (threadIdx.x == 0) *st_m = m;
}

// The blocks of a step, numbered so that no two share a number: block j of sequence b is cu_q[b] / MEMC_L + b + j.
// Returns the sequence of number x and sets the block's first token, or -1 if x is no block's number.
__device__ __forceinline__ int memory_block_of(int x, const int* __restrict__ cu_q, int n_seqs, int* base) {
  int lo = 0, hi = n_seqs - 1;  // the last b with cu_q[b] / MEMC_L + b <= x
  if (cu_q[0] / MEMC_L > x) return -1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (cu_q[mid] / MEMC_L + mid <= x) lo = mid; else hi = mid - 1;
  }
  *base = cu_q[lo] + MEMC_L * (x - (cu_q[lo] / MEMC_L + lo));
  return *base < cu_q[lo + 1] ? lo : -1;
}

// What a block's tokens weigh, for every block of the step side by side (a thread block a (block of tokens, head)):
// scores: float32 [T][heads][MEMC_L], row t: (q_t . k_s) exp(a_s - g_t) for the sources s <= t of t's block, else 0;
// wd: float32 [T][heads][2]: {exp(a_t - g_last), exp(g_c - g_t)}, the token's weight in the state after its block and
// the weight of the state before its block in the token's result.
template <typename T, int RPT>
__global__ void __launch_bounds__(MEMC_THREADS)
memory_scores_kernel(const T* __restrict__ src, long src_stride, int q_off, int k_off, float q_scale, const float* __restrict__ coef,
                     const double* __restrict__ start, const int* __restrict__ cu_q, int n_seqs, float* __restrict__ scores,
                     float* __restrict__ wd, int heads, int d) {
  constexpr int DP = MEMC_GROUPS * RPT, ROW = DP + 4;
  __shared__ __attribute__((aligned(16))) float q_s[MEMC_L][ROW];
  __shared__ __attribute__((aligned(16))) float k_s[MEMC_L][ROW];
  __shared__ double ga_s[MEMC_L], gg_s[MEMC_L];  // a and g of the block's tokens
  const int h = blockIdx.y;
  int base;
  const int b = memory_block_of(blockIdx.x, cu_q, n_seqs, &base);
  if (b < 0) return;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  const int count = min(MEMC_L, t1 - base);
  for (int x = threadIdx.x; x < MEMC_L * DP; x += MEMC_THREADS) {
    const int tok = x / DP, r = x - tok * DP;
    float qv = 0.f, kv = 0.f;
    if (tok < count && r < d) {
      const T* row = src + (size_t)(base + tok) * src_stride + (size_t)h * d + r;
      qv = Elem<T>::load(row + q_off) * q_scale, kv = Elem<T>::load(row + k_off);
    }
    q_s[tok][r] = qv, k_s[tok][r] = kv;
  }
  if (threadIdx.x < MEMC_L) {
    double a = -1e30, g = 1e30;  // a token beyond the end weighs nothing
    if ((int)threadIdx.x < count) {
      const float* cf = coef + ((size_t)(base + threadIdx.x) * heads + h) * 4;
      const double bt = *(const double*)(cf + 2);
      a = (double)cf[0] - bt, g = (double)cf[1] - bt;
    }
    ga_s[threadIdx.x] = a, gg_s[threadIdx.x] = g;
  }
  __syncthreads();
  if ((int)threadIdx.x < count) {
    double g_before = start[(size_t)b * heads + h];
    if (base > t0) {
      const float* cf = coef + ((size_t)(base - 1) * heads + h) * 4;
      g_before = (double)cf[1] - *(const double*)(cf + 2);
    }
    float* o = wd + ((size_t)(base + threadIdx.x) * heads + h) * 2;
    o[0] = expf((float)(ga_s[threadIdx.x] - gg_s[count - 1]));
    o[1] = expf((float)(g_before - gg_s[threadIdx.x]));
  }
  // a thread a token and two sources
  const int t = threadIdx.x / (MEMC_L / 2), s0 = 2 * (threadIdx.x - t * (MEMC_L / 2));
  if (t >= count) return;
  float dot0 = 0.f, dot1 = 0.f;
  if (s0 <= t) {
#pragma unroll 4
    for (int x = 0; x < DP; x += 4) {
      const float4 qq = *(const float4*)&q_s[t][x], k0 = *(const float4*)&k_s[s0][x], k1 = *(const float4*)&k_s[s0 + 1][x];
      dot0 = fmaf(qq.x, k0.x, dot0), dot0 = fmaf(qq.y, k0.y, dot0), dot0 = fmaf(qq.z, k0.z, dot0), dot0 = fmaf(qq.w, k0.w, dot0);
      dot1 = fmaf(qq.x, k1.x, dot1), dot1 = fmaf(qq.y, k1.y, dot1), dot1 = fmaf(qq.z, k1.z, dot1), dot1 = fmaf(qq.w, k1.w, dot1);
    }
    const double g = gg_s[t];
    dot0 *= expf((float)(ga_s[s0] - g));
    dot1 = s0 + 1 <= t ? dot1 * expf((float)(ga_s[s0 + 1] - g)) : 0.f;
  }
  *(float2*)(scores + ((size_t)(base + t) * heads + h) * MEMC_L + s0) = make_float2(dot0, dot1);
}

typedef float memc_acc __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float raw_to_f32(float x) { return x; }
__device__ __forceinline__ float raw_to_f32(bf16_t x) { return bf16_to_f32(x); }

// A barrier that waits for the wavefront's LDS accesses only: __syncthreads() also waits for every global load on its
// way, which here are the next block's rows, fetched early so that they arrive during this block's products.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory"); }

// y: float32 [T][heads * e], not yet divided; nq: float32 [T][heads], n_t . q_t.  TILES wavefronts a thread block, each with
// 32 rows of the block's 32 columns of S in the registers of a 32 x 32 float32 matrix instruction's result (lane l, register r:
// row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32); 32 TILES >= d.  A block of tokens takes three chains of such
// instructions a wavefront: (weighted Q) S over its rows and its share of (scores) V into one result, which the wavefronts
// add up through LDS, then K^T (weighted V) into S.  A block's q, k, v, scores and weights are fetched into registers
// while the block before is worked on.
template <typename T, int TILES>
__global__ void __launch_bounds__(CWM_WAVE * TILES)
memory_chunk_kernel(const T* __restrict__ src, long src_stride, int q_off, int k_off, int v_off, float q_scale,
                    const float* __restrict__ scores, const float* __restrict__ wd, float* __restrict__ state, long state_stride,
                    long head_elems, const int* __restrict__ cu_q, const int* __restrict__ state_slots, float* __restrict__ y,
                    float* __restrict__ nq, int heads, int d, int e, int d_pad) {
  constexpr int THREADS = CWM_WAVE * TILES, DP = 32 * TILES;
  constexpr int ROWQ = DP + 1, ROWK = DP + 4;  // a column of q across tokens, a row of k along its elements: no bank twice
  constexpr int QK_REGS = MEMC_L * DP / THREADS, V_REGS = MEMC_L * MEMC_COLS / THREADS;
  constexpr int SHARE = (MEMC_L / 2) / TILES;  // instructions of (scores) V that a wavefront issues
  __shared__ float q_s[MEMC_L][ROWQ];
  __shared__ float k_s[MEMC_L][ROWK];
  __shared__ float red[TILES][MEMC_L][MEMC_COLS];  // every wavefront's part of the block's results
  __shared__ float a_s[MEMC_L][MEMC_L + 1];        // weighted and masked scores
  __shared__ float v_s[MEMC_L][MEMC_COLS];
  __shared__ float w_s[MEMC_L], dec_s[MEMC_L];     // exp(a_s - g_last), exp(g_c - g_t)
  const int h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & (CWM_WAVE - 1), wave = threadIdx.x / CWM_WAVE;
  const int c = lane & 31, half = lane >> 5;
  const int col = blockIdx.x * MEMC_COLS + c;  // column e is the normaliser
  const int tile_row = 32 * wave;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  float* st = state + (size_t)state_slots[b] * state_stride + (size_t)h * head_elems + (size_t)col * d_pad;
  memc_acc S;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = tile_row + 8 * (r / 4) + 4 * half + (r % 4);
    S[r] = (col <= e && row < d_pad) ? st[row] : 0.f;
  }
  // What a fetch leaves in registers is what the loads return and nothing made of it: an operation on a loaded value would
  // wait for the load where the fetch is issued, not where the value is staged.  Every load is issued, from an address that
  // exists; conversion, scale and the zeros beyond the portion's end or the head's size are applied when the block is staged.
  T q_r[QK_REGS], k_r[QK_REGS], v_r[V_REGS];
  float a_r[V_REGS];
  float2 wd_r = make_float2(0.f, 0.f);
  auto fetch = [&](int base) {
    const int count = min(MEMC_L, t1 - base);
#pragma unroll
    for (int u = 0; u < QK_REGS; ++u) {
      const int x = threadIdx.x + u * THREADS, tok = x / DP, r = x - tok * DP;
      const T* row = src + (size_t)(base + min(tok, count - 1)) * src_stride + (size_t)h * d + min(r, d - 1);
      q_r[u] = row[q_off], k_r[u] = row[k_off];
    }
#pragma unroll
    for (int u = 0; u < V_REGS; ++u) {
      const int x = threadIdx.x + u * THREADS, tok = x / MEMC_COLS, cc = blockIdx.x * MEMC_COLS + (x - tok * MEMC_COLS);
      const size_t at = (size_t)(base + min(tok, count - 1));
      v_r[u] = src[at * src_stride + v_off + (size_t)h * e + min(cc, e - 1)];
      a_r[u] = scores[(at * heads + h) * MEMC_L + (x - tok * MEMC_COLS)];
    }
    wd_r = *(const float2*)(wd + ((size_t)(base + min((int)threadIdx.x, count - 1)) * heads + h) * 2);
  };
  if (t0 < t1) fetch(t0);
  for (int base = t0; base < t1; base += MEMC_L) {
    const int count = min(MEMC_L, t1 - base);
    lds_barrier();  // the block before has been read to its end
#pragma unroll
    for (int u = 0; u < QK_REGS; ++u) {
      const int x = threadIdx.x + u * THREADS, tok = x / DP, r = x - tok * DP;
      const bool live = tok < count && r < d;
      q_s[tok][r] = live ? raw_to_f32(q_r[u]) * q_scale : 0.f, k_s[tok][r] = live ? raw_to_f32(k_r[u]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < V_REGS; ++u) {
      const int x = threadIdx.x + u * THREADS, tok = x / MEMC_COLS, cl = x - tok * MEMC_COLS, cc = blockIdx.x * MEMC_COLS + cl;
      v_s[tok][cl] = tok < count ? (cc < e ? raw_to_f32(v_r[u]) : (cc == e ? 1.f : 0.f)) : 0.f;
      a_s[tok][cl] = tok < count ? a_r[u] : 0.f;
    }
    if (threadIdx.x < MEMC_L) {
      const bool live = (int)threadIdx.x < count;
      w_s[threadIdx.x] = live ? wd_r.x : 0.f, dec_s[threadIdx.x] = live ? wd_r.y : 0.f;
    }
    if (base + MEMC_L < t1) fetch(base + MEMC_L);  // on its way during this block's products
    lds_barrier();
    // what lies beyond the portion's end was staged as zeros, so every chain runs over the whole block
    memc_acc part;
#pragma unroll
    for (int r = 0; r < 16; ++r) part[r] = 0.f;
    {
      // token c of the block, as this lane's row of the left operand: the state before the block, weighted
      const float dec = dec_s[c];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float qq = dec * q_s[c][tile_row + 8 * (r / 4) + 4 * half + (r % 4)];
        part = __builtin_amdgcn_mfma_f32_32x32x2f32(qq, S[r], part, 0, 0, 0);
      }
#pragma unroll
      for (int i = wave * SHARE; i < (wave + 1) * SHARE; ++i) {
        const int s = 2 * i + half;
        part = __builtin_amdgcn_mfma_f32_32x32x2f32(a_s[c][s], v_s[s][c], part, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) red[wave][8 * (r / 4) + 4 * half + (r % 4)][c] = part[r];
    }
    {
      const float keep = dec_s[count - 1];
#pragma unroll
      for (int r = 0; r < 16; ++r) S[r] *= keep;
#pragma unroll
      for (int i = 0; i < MEMC_L / 2; ++i) {
        const int s = 2 * i + half;
        S = __builtin_amdgcn_mfma_f32_32x32x2f32(k_s[s][tile_row + c], w_s[s] * v_s[s][c], S, 0, 0, 0);
      }
    }
    lds_barrier();

    for (int x = threadIdx.x; x < MEMC_L * MEMC_COLS; x += THREADS) {
      const int t = x / MEMC_COLS, cc = x - t * MEMC_COLS, out_col = blockIdx.x * MEMC_COLS + cc;
      if (t < count && out_col <= e) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < TILES; ++w) acc += red[w][t][cc];
        if (out_col < e)
          y[(size_t)(base + t) * heads * e + (size_t)h * e + out_col] = acc;
        else
          nq[(size_t)(base + t) * heads + h] = acc;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = tile_row + 8 * (r / 4) + 4 * half + (r % 4);
    if (col <= e && row < d_pad) st[row] = S[r];
  }
}

// out[t][h * e + c] = z[t][h * e + c] / sqrt(mean_c(z[t][h]^2) + eps) * weight[h * e + c] * sigmoid(gate[t][h * e + c]);
// z = y, or, where nq is given (the results of `memory_chunk_kernel`), y / (max(|nq|, exp(-m)) + 1e-6) with m from coef;
// a wavefront a (token, head)
template <typename T>
__global__ void __launch_bounds__(MEM_THREADS)
memory_out_kernel(const float* __restrict__ y, const float* __restrict__ nq, const float* __restrict__ coef,
                  const float* __restrict__ weight, const T* __restrict__ gate, long gate_stride, T* __restrict__ out, long n_pairs,
                  int heads, int e, float eps) {
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const long pair = (long)blockIdx.x * (MEM_THREADS / CWM_WAVE) + threadIdx.x / CWM_WAVE;
  if (pair >= n_pairs) return;
  const long t = pair / heads;
  const int h = (int)(pair - t * heads);
  const float* row = y + (size_t)t * heads * e + (size_t)h * e;
  const float den = nq ? fmaxf(fabsf(nq[pair]), expf(-coef[pair * 4 + 1])) + 1e-6f : 1.0f;
  float ss = 0.f;
  for (int c = lane; c < e; c += CWM_WAVE) {
    const float z = nq ? row[c] / den : row[c];
    ss = fmaf(z, z, ss);
  }
  const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)e + eps);
  for (int c = lane; c < e; c += CWM_WAVE) {
    const float z = nq ? row[c] / den : row[c];
    const float g = Elem<T>::load(gate + (size_t)t * gate_stride + (size_t)h * e + c);
    Elem<T>::store(out + (size_t)t * heads * e + (size_t)h * e + c, z * rstd * weight[h * e + c] / (1.0f + expf(-g)));
  }
}

extern "C" int cwm_matrix_memory_block_tokens() { return MEMC_L; }

// src: the joined projection [n_tokens][src_stride] of dtype: q at column q_off (heads * d), k at k_off (heads * d), v at
// v_off (heads * e), the output gate at g_off (heads * e).  gates: float32 [n_tokens][gates_stride], the input gates'
// projection in columns 0..heads-1 and the forget gates' in heads..2 heads-1, biases included.  state: float32
// [slots][state_stride].  coef: float32 scratch [n_tokens][heads][4]; y: float32 scratch [n_tokens][heads * e].
// out: [n_tokens][heads * e] of dtype.  With `start` (float64 scratch [n_seqs][heads]), `nq` (float32 scratch
// [n_tokens][heads]) and `scores` (float32 scratch [n_tokens][heads][block tokens + 2]) the portions are taken in blocks of
// tokens; without them they are walked token by token.
extern "C" int cwm_matrix_memory(const void* src, int dtype, long src_stride, int q_off, int k_off, int v_off, int g_off,
                                 const float* gates, long gates_stride, float cap, float q_scale, float* state, long state_stride,
                                 int n_slots, const int* cu_q, const int* state_slots, int n_seqs, int n_tokens,
                                 float* coef, float* y, double* start, float* nq, float* scores, const float* weight, float eps,
                                 void* out, int heads, int d, int e, hipStream_t stream) {
  CWM_REQUIRE(heads >= 1 && d >= 1 && e >= 1 && d <= MEM_MAX_DIM, "matrix_memory: heads of %d x %d: d must lie in 1..%d", d, e, MEM_MAX_DIM);
  CWM_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && n_slots >= 1, "matrix_memory: bad counts");
  CWM_REQUIRE(cap > 0.f && eps > 0.f, "matrix_memory: the gates' cap and eps must be positive");
  const int split = mem_split(d);
  const long head_elems = cwm_matrix_memory_head_elems(d, e);
  CWM_REQUIRE(state_stride >= heads * head_elems && state_stride % 4 == 0 && ((uintptr_t)state % 16) == 0,
              "matrix_memory: a request's state needs %ld values, 16-byte aligned", heads * head_elems);
  CWM_REQUIRE(src && gates && state && cu_q && state_slots && coef && y && weight && out, "matrix_memory: arguments missing");
  CWM_REQUIRE(((uintptr_t)coef % 16) == 0, "matrix_memory: scratch must be 16-byte aligned");
  CWM_REQUIRE((start == nullptr) == (nq == nullptr) && (start == nullptr) == (scores == nullptr) && ((uintptr_t)start % 8) == 0 &&
                  ((uintptr_t)scores % 8) == 0,
              "matrix_memory: all scratch arrays of the blocked form, or none");
  if (n_seqs == 0 || n_tokens == 0) return 0;
  CWM_REQUIRE(n_seqs <= 65535, "matrix_memory: too many sequences for one launch");
  const int d_pad = MEM_ROWS * split;
  const int cols = MEM_THREADS / split;
  const int tiles = (e + cols - 1) / cols;
  const int block_tiles = (e + 1 + MEMC_COLS - 1) / MEMC_COLS;  // the normaliser is one column more
  const long n_pairs = (long)n_tokens * heads;
  const unsigned out_blocks = (unsigned)((n_pairs + MEM_THREADS / CWM_WAVE - 1) / (MEM_THREADS / CWM_WAVE));
  float* wd = scores ? scores + (size_t)n_tokens * heads * MEMC_L : nullptr;  // [n_tokens][heads][2] behind the scores
  const unsigned numbered = (unsigned)(n_tokens / MEMC_L + n_seqs);  // more than the largest number of a block of tokens
#define CWM_MEMORY_BLOCKS(T, RPT, TILES)                                                                                    \
  do {                                                                                                                      \
    hipLaunchKernelGGL((memory_scores_kernel<T, RPT>), dim3(numbered, heads), dim3(MEMC_THREADS), 0, stream, (const T*)src,  \
                       src_stride, q_off, k_off, q_scale, (const float*)coef, (const double*)start, cu_q, n_seqs, scores,   \
                       wd, heads, d);                                                                                       \
    hipLaunchKernelGGL((memory_chunk_kernel<T, TILES>), dim3(block_tiles, heads, n_seqs), dim3(CWM_WAVE * TILES), 0, stream, \
                       (const T*)src, src_stride, q_off, k_off, v_off, q_scale, (const float*)scores, (const float*)wd,     \
                       state, state_stride, head_elems, cu_q, state_slots, y, nq, heads, d, e, d_pad);                      \
  } while (0)
#define CWM_MEMORY(T)                                                                                                       \
  do {                                                                                                                      \
    if (start) {                                                                                                            \
      hipLaunchKernelGGL(memory_maxima_kernel, dim3(heads, n_seqs), dim3(MEMX_THREADS), 0, stream, gates, gates_stride, cap, \
                         state, state_stride, head_elems, cu_q, state_slots, coef, start, heads, e, d_pad);                 \
      if (d <= 32)                                                                                                          \
        CWM_MEMORY_BLOCKS(T, 4, 1);                                                                                         \
      else if (d <= 64)                                                                                                     \
        CWM_MEMORY_BLOCKS(T, 4, 2);                                                                                         \
      else if (d <= 128)                                                                                                    \
        CWM_MEMORY_BLOCKS(T, 8, 4);                                                                                         \
      else                                                                                                                  \
        CWM_MEMORY_BLOCKS(T, 16, 8);                                                                                        \
    } else {                                                                                                                \
      hipLaunchKernelGGL(memory_gates_kernel<T>, dim3(heads, n_seqs), dim3(CWM_WAVE), 0, stream, (const T*)src, src_stride,  \
                         q_off, k_off, gates, gates_stride, cap, q_scale, state, state_stride, head_elems, cu_q,            \
                         state_slots, coef, heads, d, e, d_pad);                                                            \
      hipLaunchKernelGGL(memory_scan_kernel<T>, dim3(tiles, heads, n_seqs), dim3(MEM_THREADS), 0, stream, (const T*)src,     \
                         src_stride, q_off, k_off, v_off, q_scale, (const float*)coef, state, state_stride, head_elems,     \
                         cu_q, state_slots, y, heads, d, e, split);                                                         \
    }                                                                                                                       \
    hipLaunchKernelGGL(memory_out_kernel<T>, dim3(out_blocks), dim3(MEM_THREADS), 0, stream, (const float*)y,                \
                       (const float*)nq, (const float*)coef, weight, (const T*)src + g_off, src_stride, (T*)out, n_pairs,   \
                       heads, e, eps);                                                                                      \
  } while (0)
  if (dtype == CWM_F32)
    CWM_MEMORY(float);
  else if (dtype == CWM_BF16)
    CWM_MEMORY(bf16_t);
  else
    return cwm_fail("matrix_memory: unknown type %d", dtype);
#undef CWM_MEMORY
#undef CWM_MEMORY_BLOCKS
  return cwm_launch_status("matrix_memory");
}
