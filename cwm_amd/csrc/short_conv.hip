// A short causal convolution over time on every channel, added to its own input: what a sublayer reads in place of h,
//   out_t = h_t + sum_(lag = 0 .. taps - 1) w[taps - 1 - lag] h_(t - lag)      element by element; the last tap is h_t's own
// where nothing (zero) precedes a sequence's first token.  Up to two such convolutions of the same input (two sublayers that read one
// norm's rows, each through weights of its own) are made in one pass.  The last taps - 1 inputs of a sequence are its
// state (float32 [taps - 1, D], oldest first; zero when the request is admitted), so a portion's first tokens find
// what the step before left.  `short_conv_kernel` (a thread a (token, channel)) only reads the state;
// `short_conv_state_kernel` (a thread a (sequence, channel)) replaces it afterwards, in the same stream, so no block
// waits for another.  In a step whose portions are all one token long (a decode step) the token's own thread is the
// only reader of its channel's state, and moves the rows up and appends its input itself: one launch.  float32 arithmetic; the sum runs over the taps from the oldest to the newest.
#include "common.h"

CWM_DEFINE_ERROR_API

#define SCONV_THREADS 256
#define SCONV_MAX_TAPS 16

extern "C" int cwm_short_conv_max_taps() { return SCONV_MAX_TAPS; }

template <typename T>
__global__ void __launch_bounds__(SCONV_THREADS)
short_conv_kernel(const T* __restrict__ x, long x_ld, const float* __restrict__ w1, const float* __restrict__ w2,
                  T* __restrict__ out1, T* __restrict__ out2, float* __restrict__ state, long state_ld,
                  const int* __restrict__ slots, const int* __restrict__ cu_q, const int* __restrict__ seq_of_token,
                  int n_slots, int dim, int taps, bool update_inline) {
  const int t = blockIdx.x;
  const int d = blockIdx.y * SCONV_THREADS + threadIdx.x;
  if (d >= dim) return;
  const int b = seq_of_token[t];
  const int start = cu_q[b];
  const int slot = slots[b];
  float* srow = (state && slot >= 0 && slot < n_slots) ? state + (size_t)slot * state_ld : nullptr;
  const bool moves_state = update_inline && srow && cu_q[b + 1] - start == 1;  // then t == start, and tap j reads row j
  const float own = Elem<T>::load(x + (size_t)t * x_ld + d);
  float a1 = 0.f, a2 = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int s = t - (taps - 1) + j;
    float v;
    if (s >= start)
      v = j == taps - 1 ? own : Elem<T>::load(x + (size_t)s * x_ld + d);
    else
      v = srow ? srow[(size_t)(taps - 1 + (s - start)) * dim + d] : 0.f;
    a1 = fmaf(w1[(size_t)j * dim + d], v, a1);
    if (w2) a2 = fmaf(w2[(size_t)j * dim + d], v, a2);
    if (moves_state && j >= 1) srow[(size_t)(j - 1) * dim + d] = v;  // row j - 1 was read in the round before
  }
  Elem<T>::store(out1 + (size_t)t * dim + d, own + a1);
  if (w2) Elem<T>::store(out2 + (size_t)t * dim + d, own + a2);
}

template <typename T>
__global__ void __launch_bounds__(SCONV_THREADS)
short_conv_state_kernel(const T* __restrict__ x, long x_ld, float* __restrict__ state, long state_ld,
                        const int* __restrict__ slots, const int* __restrict__ cu_q, int n_slots, int dim, int taps) {
  const int b = blockIdx.x;
  const int d = blockIdx.y * SCONV_THREADS + threadIdx.x;
  if (d >= dim) return;
  const int slot = slots[b];
  if (slot < 0 || slot >= n_slots) return;
  float* srow = state + (size_t)slot * state_ld;
  const int start = cu_q[b], n = cu_q[b + 1] - start;
  // row r of the new state is the input n - (taps - 1) + r of the portion, or, before the portion, row r + n of the
  // old state: rows are written in rising order, each after the higher row it may come from has been read
  for (int r = 0; r < taps - 1; ++r) {
    const int rel = n - (taps - 1) + r;
    const float v = rel >= 0 ? Elem<T>::load(x + (size_t)(start + rel) * x_ld + d) : srow[(size_t)(r + n) * dim + d];
    srow[(size_t)r * dim + d] = v;
  }
}

// x: [T, dim] of `dtype`, rows x_ld elements apart.  w1 (and w2, or null): float32 [taps, dim], a row a tap, the last
// row the current token's.  out1 (and out2): contiguous [T, dim] of `dtype`.  state: float32 [n_slots, state_ld] with
// (taps - 1) * dim <= state_ld (null where taps == 1); slots: int32 [n_seqs]; cu_q: int32 [n_seqs + 1]; seq_of_token:
// int32 [T].  write_state 0: the state is read and left as it was; 1: replaced by a second launch; 2: every portion of
// the step is one token long, and the first launch moves the state itself.
extern "C" int cwm_short_conv(const void* x, long x_ld, int dtype, const float* w1, const float* w2, void* out1, void* out2,
                              float* state, long state_ld, const int* slots, const int* cu_q, const int* seq_of_token,
                              int n_slots, int n_tokens, int n_seqs, int dim, int taps, int write_state, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && dim >= 1, "short_conv: bad sizes");
  CWM_REQUIRE(taps >= 1 && taps <= SCONV_MAX_TAPS, "short_conv: %d taps are outside 1..%d", taps, SCONV_MAX_TAPS);
  CWM_REQUIRE(x && w1 && out1 && (!w2 || out2) && slots && cu_q && seq_of_token, "short_conv: arguments missing");
  CWM_REQUIRE(taps == 1 || (state && state_ld >= (long)(taps - 1) * dim), "short_conv: the state does not hold %d rows of %d", taps - 1, dim);
  if (n_tokens == 0) return 0;
  const int gy = (dim + SCONV_THREADS - 1) / SCONV_THREADS;
#define CWM_SCONV(T)                                                                                                       \
  do {                                                                                                                     \
    hipLaunchKernelGGL((short_conv_kernel<T>), dim3(n_tokens, gy), dim3(SCONV_THREADS), 0, stream, (const T*)x, x_ld, w1,   \
                       w2, (T*)out1, (T*)out2, state, state_ld, slots, cu_q, seq_of_token, n_slots, dim, taps,               \
                       write_state == 2);                                                                                   \
    if (write_state == 1 && taps > 1)                                                                                      \
      hipLaunchKernelGGL((short_conv_state_kernel<T>), dim3(n_seqs, gy), dim3(SCONV_THREADS), 0, stream, (const T*)x, x_ld, \
                         state, state_ld, slots, cu_q, n_slots, dim, taps);                                                 \
  } while (0)
  if (dtype == CWM_F32) CWM_SCONV(float);
  else if (dtype == CWM_BF16) CWM_SCONV(bf16_t);
  else return cwm_fail("short_conv: unknown element type %d", dtype);
#undef CWM_SCONV
  return cwm_launch_status("short_conv");
}
