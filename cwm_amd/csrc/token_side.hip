// A layer's own input from the token: every token has a second embedding row of which each layer reads its part e
// (side_dim values), gated by the residual and added to it after a norm,
//   g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * n
// with x the float32 residual [T, D], W_gate [side_dim, D], W_proj [D, side_dim] (handed over transposed, a row a side
// value, so that neighbouring threads read neighbouring elements), n [D].  side_dim is small (tens), so
// the two products are a few dot products a token: one block a token keeps the row of x in LDS, its wavefronts take
// the gate's outputs in turn (a dot product over D each, added up by shuffles in a fixed order), then every thread
// makes elements of y from the side_dim gated values, the block adds up their squares, and the scaled row goes into
// the residual.  `round_inputs`: x and g are rounded to bfloat16 before they enter their products, as a model does
// that keeps its activations in bfloat16; the sums, the activation and the norm are float32 either way.
#include "common.h"

CWM_DEFINE_ERROR_API

#define SIDE_THREADS 256
#define SIDE_MAX_DIM 256    // side_dim
#define SIDE_MAX_WIDTH 15360

extern "C" int cwm_token_side_max_dim() { return SIDE_MAX_DIM; }
extern "C" int cwm_token_side_max_width() { return SIDE_MAX_WIDTH; }

__device__ __forceinline__ float side_round(float v, bool round) { return round ? bf16_to_f32(f32_to_bf16(v)) : v; }

template <typename TW>
__global__ void __launch_bounds__(SIDE_THREADS)
token_side_kernel(float* __restrict__ h, const int* __restrict__ tokens, const TW* __restrict__ table, long table_ld,
                  int column0, const TW* __restrict__ w_gate, const TW* __restrict__ w_proj_t, const float* __restrict__ weight,
                  int dim, int side_dim, int vocab, float eps, bool round_inputs) {
  extern __shared__ __attribute__((aligned(16))) float row[];  // [dim], then the gated values [side_dim]
  __shared__ float scratch[16];
  float* gated = row + dim;
  const int t = blockIdx.x;
  float* hrow = h + (size_t)t * dim;
  for (int e = threadIdx.x; e < dim; e += SIDE_THREADS) row[e] = side_round(hrow[e], round_inputs);
  __syncthreads();
  const int lane = threadIdx.x & (CWM_WAVE - 1), wave = threadIdx.x / CWM_WAVE;
  const int token = tokens[t];
  const bool known = token >= 0 && token < vocab;
  for (int k = wave; k < side_dim; k += SIDE_THREADS / CWM_WAVE) {
    const TW* wrow = w_gate + (size_t)k * dim;
    float a = 0.f;
    for (int e = lane; e < dim; e += CWM_WAVE) a = fmaf(Elem<TW>::load(wrow + e), row[e], a);
    a = wave_sum(a);
    if (lane == 0) {
      const float z = side_round(a, round_inputs);
      const float gelu = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
      const float e_k = known ? Elem<TW>::load(table + (size_t)token * table_ld + column0 + k) : __uint_as_float(0x7fc00000u);
      gated[k] = side_round(gelu * e_k, round_inputs);
    }
  }
  __syncthreads();
  // y stays in registers: a thread's elements are e = threadIdx.x + i * SIDE_THREADS
  constexpr int MAXE = SIDE_MAX_WIDTH / SIDE_THREADS;
  float y[MAXE];
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < MAXE; ++i) {
    const int e = threadIdx.x + i * SIDE_THREADS;
    y[i] = 0.f;
    if (e < dim) {
      float a = 0.f;
      for (int k = 0; k < side_dim; ++k) a = fmaf(Elem<TW>::load(w_proj_t + (size_t)k * dim + e), gated[k], a);
      y[i] = a;
      sq += a * a;
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(sq, scratch) / (float)dim + eps);
#pragma unroll
  for (int i = 0; i < MAXE; ++i) {
    const int e = threadIdx.x + i * SIDE_THREADS;
    if (e < dim) hrow[e] += y[i] * rstd * weight[e];
  }
}

// h: float32 [T, dim], changed in place.  tokens: int32 [T].  table: [vocab, >= column0 + side_dim] of `w_dtype`, rows
// table_ld apart; w_gate [side_dim, dim] and w_proj_t [side_dim, dim] (the projection transposed) of `w_dtype`, contiguous;
// weight: float32 [dim].
extern "C" int cwm_token_side(float* h, const int* tokens, const void* table, long table_ld, int column0, const void* w_gate,
                              const void* w_proj_t, int w_dtype, const float* weight, int n_tokens, int dim, int side_dim, int vocab,
                              float eps, int round_inputs, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && vocab >= 1 && column0 >= 0, "token_side: bad sizes");
  CWM_REQUIRE(dim >= 1 && dim <= SIDE_MAX_WIDTH, "token_side: rows of %d elements are outside 1..%d", dim, SIDE_MAX_WIDTH);
  CWM_REQUIRE(side_dim >= 1 && side_dim <= SIDE_MAX_DIM, "token_side: %d side values are outside 1..%d", side_dim, SIDE_MAX_DIM);
  CWM_REQUIRE(h && tokens && table && w_gate && w_proj_t && weight, "token_side: arguments missing");
  CWM_REQUIRE(eps > 0.f, "token_side: eps must be positive");
  if (n_tokens == 0) return 0;
  const size_t lds = sizeof(float) * ((size_t)dim + side_dim);
#define CWM_SIDE(TW)                                                                                                    \
  hipLaunchKernelGGL((token_side_kernel<TW>), dim3(n_tokens), dim3(SIDE_THREADS), lds, stream, h, tokens, (const TW*)table, \
                     table_ld, column0, (const TW*)w_gate, (const TW*)w_proj_t, weight, dim, side_dim, vocab, eps, round_inputs != 0)
  if (w_dtype == CWM_F32) CWM_SIDE(float);
  else if (w_dtype == CWM_BF16) CWM_SIDE(bf16_t);
  else return cwm_fail("token_side: unknown element type %d", w_dtype);
#undef CWM_SIDE
  return cwm_launch_status("token_side");
}
