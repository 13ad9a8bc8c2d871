// Gated linear attention: a matrix state per head that decays channel by channel.
//
//   alpha_t = sigmoid(z_t)^(1 / tau)                     one decay a key channel (z: float32 logits, heads x dim)
//   S_t     = diag(alpha_t) S_(t-1) + k_t v_t^T          S: dim x vdim, float32, carried from token to token
//   o_t     = S_t^T (q_scale q_t)
//   out_t   = o_t / sqrt(mean(o_t^2) + eps) * w * silu(g_t)     per head over vdim; w of vdim values for all heads
//
// `gla_walk_kernel`: a block a (tile of value columns, head, sequence) walks the sequence's tokens of the step one by
// one, from the state that the step before left in the sequence's slot, and leaves the new state there.  A thread
// holds up to 32 rows of one column of S in registers; `split` neighbouring lanes share a column (a run of consecutive
// rows each, a multiple of four, read from LDS sixteen bytes at a time) and add their parts of o_t by shuffles.  q, k, the decays and v of 16 (or 8) tokens are staged in LDS at a time,
// in float32, the decays computed once a (token, channel).  The same tokens give the same bits however they are cut
// into steps.  The state of a (head, tile) lies in memory in the order its threads hold it (row r of thread i at
// [r][i]), so it is read and written in whole lines; only this kernel looks inside.
// A step with a portion of more than a segment of tokens runs all its portions in segments side by side, in three
// launches: every segment but a sequence's last from a zero state, leaving its own sum and the product of its decays
// (MODE 1); `gla_carry_kernel`, which carries the states across a sequence's segments, start_(s+1) = decay_s *
// start_s + sum_s; and every segment from its true start with its results (MODE 2).  That differs from the walk by
// float32 rounding only.
// `gla_out_kernel`: the norm of every head's o_t, its weight and the gate, a wavefront a (token, head).
#include "common.h"

CWM_DEFINE_ERROR_API

#define GLA_THREADS 256
#define GLA_ROWS 32        // rows of a column that one thread holds at most
#define GLA_MAX_DIM 256    // = GLA_ROWS * 8 lanes a column
#define GLA_CHUNK 16       // tokens staged at a time (8 where the rows are long)

extern "C" int cwm_gla_max_dim() { return GLA_MAX_DIM; }

// lanes that share a column of the state: the fewest (1, 2, 4, 8) that leave a lane at most GLA_ROWS rows
static inline int gla_split(int dim) {
  int split = 1;
  while (split < 8 && (dim + split - 1) / split > GLA_ROWS) split *= 2;
  return split;
}
// rows of a column that a lane holds: a multiple of 4
static inline int gla_rows(int dim, int split) { return ((dim + split - 1) / split + 3) / 4 * 4; }
extern "C" int cwm_gla_split(int dim) { return gla_split(dim); }
// float32 elements of a request's state
extern "C" long cwm_gla_state_elems(int heads, int dim, int vdim) {
  const int split = gla_split(dim), rows = gla_rows(dim, split), cols = GLA_THREADS / split;
  return (long)heads * ((vdim + cols - 1) / cols) * rows * GLA_THREADS;
}

__device__ __forceinline__ int gla_rows_device(int dim, int split) { return ((dim + split - 1) / split + 3) / 4 * 4; }

__device__ __forceinline__ float gla_decay(float z, float inv_tau) {
  // sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau), with softplus(x) = max(x, 0) + log1p(exp(-|x|))
  const float sp = fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)));
  return expf(-sp * inv_tau);
}

// segments: int32 [n][6]: sequence, first token, end token, number of the segment in its sequence, the sequence's first
// entry of the scratch states, segments of the sequence.
// MODE 0: a block a (tile, head, sequence) walks the sequence's tokens from the state in its slot and leaves the new one.
// MODE 1: a block a (tile, head, segment) walks from zero without results and leaves the segment's sum and decay product.
// MODE 2: a block a (tile, head, segment) walks from seg_start with results; a sequence's last segment writes the slot.
template <typename T, int MODE>
__global__ void __launch_bounds__(GLA_THREADS)
gla_walk_kernel(const T* __restrict__ proj, long proj_ld, const float* __restrict__ z, long z_ld, float* __restrict__ o_raw,
                float* __restrict__ state, long state_ld, const int* __restrict__ slots, const int* __restrict__ cu_q,
                int n_slots, int heads, int dim, int vdim, int split, int chunk, float inv_tau, float q_scale,
                const int* __restrict__ segments, float* __restrict__ seg_local, float* __restrict__ seg_decay,
                const float* __restrict__ seg_start, long seg_ld) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int vt = blockIdx.x, h = blockIdx.y;
  const int cols = GLA_THREADS / split, rows = gla_rows_device(dim, split), dpad = split * rows;
  const int col = threadIdx.x / split, part = threadIdx.x % split;
  const int e = vt * cols + col;  // this thread's value column
  const bool live = e < vdim;
  float* qs = lds;                  // [chunk][dpad]: rows beyond dim hold zeros (a zero key and query leave their rows of S at zero)
  float* ks = qs + chunk * dpad;    // [chunk][dpad]
  float* as = ks + chunk * dpad;    // [chunk][dpad]
  float* vs = as + chunk * dpad;    // [chunk][cols]
  int b, t0, t1, seg = 0;
  bool last = true;
  if constexpr (MODE == 0) {
    b = blockIdx.z, t0 = cu_q[b], t1 = cu_q[b + 1];
  } else {
    const int* sg = segments + 6 * blockIdx.z;
    b = sg[0], t0 = sg[1], t1 = sg[2], seg = sg[4] + sg[3], last = sg[3] == sg[5] - 1;
    if (MODE == 1 && last) return;  // nothing comes after it
  }
  const int slot = slots[b];
  if (slot < 0 || slot >= n_slots) return;
  const int n_vt = gridDim.x;
  const size_t tile_at = ((size_t)h * n_vt + vt) * rows * GLA_THREADS + threadIdx.x;
  float* st = state + (size_t)slot * state_ld + tile_at;
  float S[GLA_ROWS];
  float P[MODE == 1 ? GLA_ROWS : 1];
#pragma unroll
  for (int r = 0; r < GLA_ROWS; ++r) {
    if constexpr (MODE == 0) S[r] = r < rows ? st[(size_t)r * GLA_THREADS] : 0.f;
    if constexpr (MODE == 1) S[r] = 0.f, P[r] = 1.f;
    if constexpr (MODE == 2) S[r] = r < rows ? seg_start[(size_t)seg * seg_ld + tile_at + (size_t)r * GLA_THREADS] : 0.f;
  }
  const int q_off = h * dim, k_off = heads * dim + h * dim, v_off = 2 * heads * dim + h * vdim;
  for (int c0 = t0; c0 < t1; c0 += chunk) {
    const int n = min(chunk, t1 - c0);
    __syncthreads();  // the chunk before has been walked
    for (int i = threadIdx.x; i < n * dpad; i += GLA_THREADS) {
      const int tt = i / dpad, d = i - tt * dpad;
      const T* row = proj + (size_t)(c0 + tt) * proj_ld;
      const bool real = d < dim;
      if constexpr (MODE != 1) qs[i] = real ? Elem<T>::load(row + q_off + d) * q_scale : 0.f;
      ks[i] = real ? Elem<T>::load(row + k_off + d) : 0.f;
      as[i] = real ? gla_decay(z[(size_t)(c0 + tt) * z_ld + h * dim + d], inv_tau) : 0.f;
    }
    for (int i = threadIdx.x; i < n * cols; i += GLA_THREADS) {
      const int tt = i / cols, cc = i - tt * cols;
      const int ee = vt * cols + cc;
      vs[i] = ee < vdim ? Elem<T>::load(proj + (size_t)(c0 + tt) * proj_ld + v_off + ee) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float v = vs[tt * cols + col];
      const float* qrow = qs + tt * dpad;
      const float* krow = ks + tt * dpad;
      const float* arow = as + tt * dpad;
      float o = 0.f;
      const int d0 = part * rows;  // this lane's rows: d0 .. d0 + rows - 1 (rows is a multiple of 4; LDS rows are padded to it)
#pragma unroll
      for (int r = 0; r < GLA_ROWS; r += 4) {
        if (r < rows) {
          const float4 a4 = *(const float4*)(arow + d0 + r);
          const float4 k4 = *(const float4*)(krow + d0 + r);
          S[r] = fmaf(a4.x, S[r], k4.x * v), S[r + 1] = fmaf(a4.y, S[r + 1], k4.y * v);
          S[r + 2] = fmaf(a4.z, S[r + 2], k4.z * v), S[r + 3] = fmaf(a4.w, S[r + 3], k4.w * v);
          if constexpr (MODE == 1) P[r] *= a4.x, P[r + 1] *= a4.y, P[r + 2] *= a4.z, P[r + 3] *= a4.w;
          if constexpr (MODE != 1) {
            const float4 q4 = *(const float4*)(qrow + d0 + r);
            o = fmaf(S[r], q4.x, o), o = fmaf(S[r + 1], q4.y, o), o = fmaf(S[r + 2], q4.z, o), o = fmaf(S[r + 3], q4.w, o);
          }
        }
      }
      if constexpr (MODE != 1) {
        for (int off = 1; off < split; off *= 2) o += __shfl_xor(o, off, CWM_WAVE);
        if (part == 0 && live) o_raw[(size_t)(c0 + tt) * heads * vdim + h * vdim + e] = o;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < GLA_ROWS; ++r) {
    if (r >= rows) continue;
    if constexpr (MODE == 1) {
      seg_local[(size_t)seg * seg_ld + tile_at + (size_t)r * GLA_THREADS] = S[r];
      seg_decay[(size_t)seg * seg_ld + tile_at + (size_t)r * GLA_THREADS] = P[r];
    } else {
      if (last) st[(size_t)r * GLA_THREADS] = S[r];
    }
  }
}

// The states at the segments' starts: a thread an element of the state walks the step's segments in their order.
__global__ void __launch_bounds__(GLA_THREADS)
gla_carry_kernel(const int* __restrict__ segments, int n_segments, const float* __restrict__ state, long state_ld,
                 const int* __restrict__ slots, int n_slots, const float* __restrict__ seg_local,
                 const float* __restrict__ seg_decay, float* __restrict__ seg_start, long seg_ld, long elems) {
  const long i = (long)blockIdx.x * GLA_THREADS + threadIdx.x;
  if (i >= elems) return;
  float cur = 0.f;
  for (int s = 0; s < n_segments; ++s) {
    const int* sg = segments + 6 * s;
    const int seg = sg[4] + sg[3];
    if (sg[3] == 0) {
      const int slot = slots[sg[0]];
      cur = (slot >= 0 && slot < n_slots) ? state[(size_t)slot * state_ld + i] : 0.f;
    }
    seg_start[(size_t)seg * seg_ld + i] = cur;
    if (sg[3] < sg[5] - 1) cur = fmaf(seg_decay[(size_t)seg * seg_ld + i], cur, seg_local[(size_t)seg * seg_ld + i]);
  }
}

template <typename T>
__global__ void __launch_bounds__(CWM_WAVE)
gla_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate, long gate_ld, const float* __restrict__ weight,
               T* __restrict__ out, int heads, int vdim, float eps) {
  const int t = blockIdx.x / heads, h = blockIdx.x - t * heads;
  const float* o = o_raw + ((size_t)t * heads + h) * vdim;
  float sq = 0.f;
  for (int e = threadIdx.x; e < vdim; e += CWM_WAVE) sq += o[e] * o[e];
  const float rstd = 1.0f / sqrtf(wave_sum(sq) / (float)vdim + eps);
  for (int e = threadIdx.x; e < vdim; e += CWM_WAVE) {
    const float g = Elem<T>::load(gate + (size_t)t * gate_ld + h * vdim + e);
    const float y = o[e] * rstd * weight[e] * (g / (1.0f + expf(-g)));
    Elem<T>::store(out + ((size_t)t * heads + h) * vdim + e, y);
  }
}

// proj: [T, >= 2 * heads * dim + 2 * heads * vdim] of `dtype`, rows proj_ld elements apart: q, k (heads x dim each),
// v, g (heads x vdim each).  z: float32 [T, heads * dim], rows z_ld apart.  weight: float32 [vdim].  state: float32
// [n_slots, state_ld] with cwm_gla_state_elems(...) <= state_ld elements a request; slots: int32 [n_seqs]; cu_q: int32
// [n_seqs + 1].  o_raw: float32 [T, heads * vdim] scratch.  out: [T, heads * vdim] of `dtype`.  segments (or null: every
// sequence is walked by one block a tile): int32 [n_segments][6] as above, all segments of the step in the order of the
// sequences; seg_local, seg_decay, seg_start: float32 [n_segments][seg_ld] scratch.
extern "C" int cwm_gated_linear_attention(const void* proj, long proj_ld, int dtype, const float* z, long z_ld,
                                          const float* weight, float* o_raw, void* out, float* state, long state_ld,
                                          const int* slots, const int* cu_q, int n_slots, int n_tokens, int n_seqs, int heads,
                                          int dim, int vdim, float tau, float eps, float q_scale, const int* segments,
                                          int n_segments, float* seg_local, float* seg_decay, float* seg_start, long seg_ld,
                                          hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && heads >= 1 && vdim >= 1, "gated_linear_attention: bad sizes");
  CWM_REQUIRE(dim >= 1 && dim <= GLA_MAX_DIM, "gated_linear_attention: heads of %d rows are outside 1..%d", dim, GLA_MAX_DIM);
  CWM_REQUIRE(tau > 0.f && eps > 0.f, "gated_linear_attention: tau and eps must be positive");
  CWM_REQUIRE(proj && z && weight && o_raw && out && state && slots && cu_q, "gated_linear_attention: arguments missing");
  CWM_REQUIRE(state_ld >= cwm_gla_state_elems(heads, dim, vdim), "gated_linear_attention: a state row of %ld elements is too short", state_ld);
  CWM_REQUIRE(n_seqs <= 65535 && heads <= 65535 && n_segments <= 65535, "gated_linear_attention: too many sequences, segments or heads for one launch");
  CWM_REQUIRE(!segments || (n_segments >= 1 && seg_local && seg_decay && seg_start && seg_ld >= cwm_gla_state_elems(heads, dim, vdim)),
              "gated_linear_attention: segments need their scratch states");
  if (n_tokens == 0 || n_seqs == 0) return 0;
  const int split = gla_split(dim), cols = GLA_THREADS / split, n_vt = (vdim + cols - 1) / cols;
  const int dpad = split * gla_rows(dim, split);
  int chunk = GLA_CHUNK;
  while (chunk > 1 && sizeof(float) * (size_t)chunk * (3 * dpad + cols) > 49152) chunk /= 2;
  const size_t lds = sizeof(float) * (size_t)chunk * (3 * dpad + cols);
  const dim3 grid(n_vt, heads, n_seqs), grid_seg(n_vt, heads, segments ? n_segments : 1);
  const long elems = cwm_gla_state_elems(heads, dim, vdim);
  const float inv_tau = 1.0f / tau;
#define CWM_GLA_WALK(T, MODE, GRID)                                                                                         \
  hipLaunchKernelGGL((gla_walk_kernel<T, MODE>), GRID, dim3(GLA_THREADS), lds, stream, (const T*)proj, proj_ld, z, z_ld, o_raw, \
                     state, state_ld, slots, cu_q, n_slots, heads, dim, vdim, split, chunk, inv_tau, q_scale, segments, seg_local, \
                     seg_decay, seg_start, seg_ld)
#define CWM_GLA(T)                                                                                                         \
  do {                                                                                                                     \
    if (segments) {                                                                                                        \
      CWM_GLA_WALK(T, 1, grid_seg);                                                                                        \
      hipLaunchKernelGGL(gla_carry_kernel, dim3((unsigned)((elems + GLA_THREADS - 1) / GLA_THREADS)), dim3(GLA_THREADS), 0,  \
                         stream, segments, n_segments, state, state_ld, slots, n_slots, seg_local, seg_decay, seg_start,     \
                         seg_ld, elems);                                                                                     \
      CWM_GLA_WALK(T, 2, grid_seg);                                                                                        \
    } else {                                                                                                               \
      CWM_GLA_WALK(T, 0, grid);                                                                                            \
    }                                                                                                                      \
    hipLaunchKernelGGL((gla_out_kernel<T>), dim3(n_tokens * heads), dim3(CWM_WAVE), 0, stream, o_raw,                        \
                       (const T*)proj + 2 * (size_t)heads * dim + (size_t)heads * vdim, proj_ld, weight, (T*)out, heads,     \
                       vdim, eps);                                                                                           \
  } while (0)
  if (dtype == CWM_F32) CWM_GLA(float);
  else if (dtype == CWM_BF16) CWM_GLA(bf16_t);
  else return cwm_fail("gated_linear_attention: unknown element type %d", dtype);
#undef CWM_GLA
#undef CWM_GLA_WALK
  return cwm_launch_status("gated_linear_attention");
}
