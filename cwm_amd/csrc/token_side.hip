// A layer's own input from the token: every token has a second embedding row of which each layer reads its part e
// (side_dim values), gated by the residual and added to it after a norm,
//   g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * n
// with x the float32 residual [T, D], W_gate [side_dim, D], W_proj [D, side_dim] (handed over transposed, a row a side
// value, so that neighbouring threads read neighbouring elements), n [D].  side_dim is small (tens), so
// the two products are a few dot products a token: one block a token keeps the row of x in LDS, its wavefronts take
// the gate's outputs in turn (a dot product over D each, added up by shuffles in a fixed order), then every thread
// makes elements of y from the side_dim gated values, the block adds up their squares, and the scaled row goes into
// the residual (several tokens a block where the step has many, so that the matrices are read once for all of them).
// `round_inputs`: x and g are rounded to bfloat16 before they enter their products, as a model does
// that keeps its activations in bfloat16; the sums, the activation and the norm are float32 either way.
#include "common.h"

CWM_DEFINE_ERROR_API

#define SIDE_THREADS 1024
#define SIDE_MAX_DIM 256    // side_dim
#define SIDE_MAX_WIDTH 15360
#define SIDE_LDS_LIMIT 61440
#define SIDE_GATE_ROWS 4   // rows of the gate that a wavefront reads side by side
#define SIDE_MAX_ADDENDS 4

// What is still to be added to the residual before the input is made (the layer's sublayers' results): each addend a
// [T, D] tensor (rows may lie apart) or float32 partial sums [P, T, D], times a constant; added in their order, in
// float32, the partial sums of an addend first among themselves, as the layer norm kernel adds them.
struct SideAddend {
  const void* ptr;
  long ld;              // elements between rows
  long partial_stride;  // elements between partial sums
  int n_partials;
  int dtype;
  float scale;
};

struct SideAddends {
  SideAddend a[SIDE_MAX_ADDENDS];
  int n;
};

extern "C" int cwm_token_side_max_addends() { return SIDE_MAX_ADDENDS; }

extern "C" int cwm_token_side_max_dim() { return SIDE_MAX_DIM; }
extern "C" int cwm_token_side_max_width() { return SIDE_MAX_WIDTH; }

__device__ __forceinline__ float side_round(float v, bool round) { return round ? bf16_to_f32(f32_to_bf16(v)) : v; }

template <typename T> struct SideVec;
template <> struct SideVec<bf16_t> {
  static constexpr int N = 8;  // elements of a 16-byte load
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 x = *(const uint4*)p;
    v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
    v[4] = __uint_as_float(x.z << 16), v[5] = __uint_as_float(x.z & 0xffff0000u);
    v[6] = __uint_as_float(x.w << 16), v[7] = __uint_as_float(x.w & 0xffff0000u);
  }
};
template <> struct SideVec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  }
};

// TOK tokens a block: the two matrices are read once for all of them.  The gate's rows are dealt to the block's
// wavefronts, which read them 16 bytes a lane; every sum runs in one order whatever TOK is.
template <typename TW, int TOK>
__global__ void __launch_bounds__(SIDE_THREADS)
token_side_kernel(float* __restrict__ h, const int* __restrict__ tokens, const TW* __restrict__ table, long table_ld,
                  int column0, const TW* __restrict__ w_gate, const TW* __restrict__ w_proj_t, const float* __restrict__ weight,
                  int n_tokens, int dim, int side_dim, int vocab, float eps, bool round_inputs, SideAddends addends) {
  extern __shared__ __attribute__((aligned(16))) float rows[];  // [TOK][dim], then the gated values [TOK][side_dim]
  __shared__ float scratch[16];
  float* gated = rows + (size_t)TOK * dim;
  const int t0 = blockIdx.x * TOK;
  for (int e = threadIdx.x; e < TOK * dim; e += SIDE_THREADS) {
    const int tok = e / dim, el = e - tok * dim;
    const size_t t = (size_t)t0 + tok;
    float x = 0.f;
    if (t < (size_t)n_tokens) {
      x = h[t * dim + el];
      for (int a = 0; a < addends.n; ++a) {
        const SideAddend& ad = addends.a[a];
        float y = 0.f;
        for (int p = 0; p < ad.n_partials; ++p) {
          const size_t at = (size_t)p * ad.partial_stride + t * ad.ld + el;
          y += ad.dtype == CWM_F32 ? ((const float*)ad.ptr)[at] : bf16_to_f32(((const bf16_t*)ad.ptr)[at]);
        }
        x = fmaf(ad.scale, y, x);
      }
      if (addends.n > 0) h[t * dim + el] = x;  // read again at the end, after the block's barriers
    }
    rows[e] = side_round(x, round_inputs);
  }
  __syncthreads();
  const int lane = threadIdx.x & (CWM_WAVE - 1), wave = threadIdx.x / CWM_WAVE;
  constexpr int N = SideVec<TW>::N;
  const bool vec = dim % N == 0 && ((uintptr_t)w_gate % 16) == 0;
  // a wavefront takes SIDE_GATE_ROWS rows of the gate at a time, so that as many loads are in flight
  for (int k0 = wave * SIDE_GATE_ROWS; k0 < side_dim; k0 += (SIDE_THREADS / CWM_WAVE) * SIDE_GATE_ROWS) {
    float a[SIDE_GATE_ROWS][TOK];
#pragma unroll
    for (int kk = 0; kk < SIDE_GATE_ROWS; ++kk)
#pragma unroll
      for (int tok = 0; tok < TOK; ++tok) a[kk][tok] = 0.f;
    if (vec) {
      for (int e0 = lane * N; e0 < dim; e0 += CWM_WAVE * N) {
        float w[SIDE_GATE_ROWS][N];
#pragma unroll
        for (int kk = 0; kk < SIDE_GATE_ROWS; ++kk) SideVec<TW>::load(w_gate + (size_t)min(k0 + kk, side_dim - 1) * dim + e0, w[kk]);
#pragma unroll
        for (int tok = 0; tok < TOK; ++tok)
#pragma unroll
          for (int i = 0; i < N; ++i) {
            const float x = rows[tok * dim + e0 + i];
#pragma unroll
            for (int kk = 0; kk < SIDE_GATE_ROWS; ++kk) a[kk][tok] = fmaf(w[kk][i], x, a[kk][tok]);
          }
      }
    } else {
      for (int e = lane; e < dim; e += CWM_WAVE) {
#pragma unroll
        for (int kk = 0; kk < SIDE_GATE_ROWS; ++kk) {
          const float w = Elem<TW>::load(w_gate + (size_t)min(k0 + kk, side_dim - 1) * dim + e);
#pragma unroll
          for (int tok = 0; tok < TOK; ++tok) a[kk][tok] = fmaf(w, rows[tok * dim + e], a[kk][tok]);
        }
      }
    }
#pragma unroll
    for (int kk = 0; kk < SIDE_GATE_ROWS; ++kk) {
      const int k = k0 + kk;
#pragma unroll
      for (int tok = 0; tok < TOK; ++tok) {
        const float sum = wave_sum(a[kk][tok]);
        if (lane == 0 && k < side_dim && t0 + tok < n_tokens) {
          const float z = side_round(sum, round_inputs);
          const float gelu = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
          const int token = tokens[t0 + tok];
          const bool known = token >= 0 && token < vocab;
          const float e_k = known ? Elem<TW>::load(table + (size_t)token * table_ld + column0 + k) : __uint_as_float(0x7fc00000u);
          gated[tok * side_dim + k] = side_round(gelu * e_k, round_inputs);
        }
      }
    }
  }
  __syncthreads();
  // y stays in registers: a thread's elements are e = threadIdx.x + i * SIDE_THREADS
  constexpr int MAXE = SIDE_MAX_WIDTH / SIDE_THREADS;
  float y[TOK][MAXE];
  float sq[TOK];
#pragma unroll
  for (int tok = 0; tok < TOK; ++tok) sq[tok] = 0.f;
#pragma unroll
  for (int i = 0; i < MAXE; ++i) {
    const int e = threadIdx.x + i * SIDE_THREADS;
#pragma unroll
    for (int tok = 0; tok < TOK; ++tok) y[tok][i] = 0.f;
    if (e < dim) {
#pragma unroll 8
      for (int k = 0; k < side_dim; ++k) {
        const float w = Elem<TW>::load(w_proj_t + (size_t)k * dim + e);
#pragma unroll
        for (int tok = 0; tok < TOK; ++tok) y[tok][i] = fmaf(w, gated[tok * side_dim + k], y[tok][i]);
      }
#pragma unroll
      for (int tok = 0; tok < TOK; ++tok) sq[tok] += y[tok][i] * y[tok][i];
    }
  }
#pragma unroll
  for (int tok = 0; tok < TOK; ++tok) {
    const float rstd = 1.0f / sqrtf(block_sum(sq[tok], scratch) / (float)dim + eps);
    if (t0 + tok < n_tokens) {
      float* hrow = h + (size_t)(t0 + tok) * dim;
#pragma unroll
      for (int i = 0; i < MAXE; ++i) {
        const int e = threadIdx.x + i * SIDE_THREADS;
        if (e < dim) hrow[e] += y[tok][i] * rstd * weight[e];
      }
    }
  }
}

// h: float32 [T, dim], changed in place.  Addend a (n_addends of them, or none): ptrs[a] of dtypes[a], rows lds[a]
// elements apart, n_partials[a] slabs partial_strides[a] elements apart, times scales[a]; they are added to h first.
// tokens: int32 [T].  table: [vocab, >= column0 + side_dim] of `w_dtype`, rows
// table_ld apart; w_gate [side_dim, dim] and w_proj_t [side_dim, dim] (the projection transposed) of `w_dtype`, contiguous;
// weight: float32 [dim].
extern "C" int cwm_token_side(float* h, const int* tokens, const void* table, long table_ld, int column0, const void* w_gate,
                              const void* w_proj_t, int w_dtype, const float* weight, int n_tokens, int dim, int side_dim, int vocab,
                              float eps, int round_inputs, int n_addends, const void* const* ptrs, const int* dtypes,
                              const long* lds_, const int* n_partials, const long* partial_strides, const float* scales,
                              hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && vocab >= 1 && column0 >= 0, "token_side: bad sizes");
  CWM_REQUIRE(dim >= 1 && dim <= SIDE_MAX_WIDTH, "token_side: rows of %d elements are outside 1..%d", dim, SIDE_MAX_WIDTH);
  CWM_REQUIRE(side_dim >= 1 && side_dim <= SIDE_MAX_DIM, "token_side: %d side values are outside 1..%d", side_dim, SIDE_MAX_DIM);
  CWM_REQUIRE(h && tokens && table && w_gate && w_proj_t && weight, "token_side: arguments missing");
  CWM_REQUIRE(eps > 0.f, "token_side: eps must be positive");
  CWM_REQUIRE(n_addends >= 0 && n_addends <= SIDE_MAX_ADDENDS, "token_side: %d addends, at most %d are taken", n_addends, SIDE_MAX_ADDENDS);
  if (n_tokens == 0) return 0;
  SideAddends ad;
  ad.n = n_addends;
  for (int a = 0; a < n_addends; ++a) {
    CWM_REQUIRE(ptrs[a] && n_partials[a] >= 1, "token_side: addend %d is empty", a);
    CWM_REQUIRE(n_partials[a] == 1 || dtypes[a] == CWM_F32, "token_side: partial sums must be float32");
    ad.a[a] = SideAddend{ptrs[a], lds_[a], partial_strides[a], n_partials[a], dtypes[a], scales[a]};
  }
  // tokens a block: as many (4, 2, 1) as fit the LDS and still leave the chip a block a few tokens
  int tok = 4;
  while (tok > 1 && (sizeof(float) * (size_t)tok * (dim + side_dim) > SIDE_LDS_LIMIT || n_tokens < 64 * tok)) tok /= 2;
  CWM_REQUIRE(sizeof(float) * ((size_t)dim + side_dim) <= SIDE_LDS_LIMIT, "token_side: a row of %d and %d side values do not fit the LDS", dim, side_dim);
  const size_t lds = sizeof(float) * (size_t)tok * (dim + side_dim);
  const int blocks = (n_tokens + tok - 1) / tok;
#define CWM_SIDE_TOK(TW, TOK)                                                                                            \
  hipLaunchKernelGGL((token_side_kernel<TW, TOK>), dim3(blocks), dim3(SIDE_THREADS), lds, stream, h, tokens, (const TW*)table, \
                     table_ld, column0, (const TW*)w_gate, (const TW*)w_proj_t, weight, n_tokens, dim, side_dim, vocab, eps, round_inputs != 0, ad)
#define CWM_SIDE(TW)                            \
  do {                                          \
    if (tok == 4) CWM_SIDE_TOK(TW, 4);          \
    else if (tok == 2) CWM_SIDE_TOK(TW, 2);     \
    else CWM_SIDE_TOK(TW, 1);                   \
  } while (0)
  if (w_dtype == CWM_F32) CWM_SIDE(float);
  else if (w_dtype == CWM_BF16) CWM_SIDE(bf16_t);
  else return cwm_fail("token_side: unknown element type %d", w_dtype);
#undef CWM_SIDE
#undef CWM_SIDE_TOK
  return cwm_launch_status("token_side");
}
