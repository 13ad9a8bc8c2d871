// Layer norm (mean and variance over a row, weight and bias) fused with the residual sum that precedes it, for
// layers whose sublayers all read the same residual: x <- x + sum_a c_a y_a, then up to two normalised copies of
// the new x that share its mean and variance,
//     out_i = (x - mean) / sqrt(var + eps) * w_i + b_i,      var = mean((x - mean)^2).
// Each addend y_a is a [T, D] tensor (rows may lie apart) or float32 partial sums [P, T, D] of a product whose K
// was split, added in order; c_a is a constant.  The sum, the statistics and the norm are float32; the addends are
// added in the order they are given, after the residual.  One block a row; the row stays in LDS between the passes
// (the variance is taken about the mean, in a second pass).  With `rows` only those rows are normalised and the
// residual is left as it was.
#include "common.h"

CWM_DEFINE_ERROR_API

#define LN_MAX_ADDENDS 4
#define LN_MAX_DIM 15360  // the row lies in LDS beside the reductions' scratch, within 64 KB
#define LN_THREADS 256

struct LnAddend {
  const void* ptr;
  long ld;              // elements between rows
  long partial_stride;  // elements between partial sums
  int n_partials;
  int dtype;
  float scale;
};

struct LnAddends {
  LnAddend a[LN_MAX_ADDENDS];
  int n;
};

extern "C" int cwm_layernorm_max_addends() { return LN_MAX_ADDENDS; }
extern "C" int cwm_layernorm_max_dim() { return LN_MAX_DIM; }

__device__ __forceinline__ void ln_load4(const void* p, int dtype, size_t e, float (&v)[4]) {
  if (dtype == CWM_F32) {
    const float4 x = *(const float4*)((const float*)p + e);
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  } else {
    const uint2 x = *(const uint2*)((const bf16_t*)p + e);
    v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
}

__device__ __forceinline__ float ln_load1(const void* p, int dtype, size_t e) {
  return dtype == CWM_F32 ? ((const float*)p)[e] : bf16_to_f32(((const bf16_t*)p)[e]);
}

template <typename TO> struct LnStore;
template <> struct LnStore<float> {
  static __device__ __forceinline__ void four(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct LnStore<bf16_t> {
  static __device__ __forceinline__ void four(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = pack2_bf16(v[0], v[1]);
    x.y = pack2_bf16(v[2], v[3]);
    *(uint2*)p = x;
  }
};

// VEC: D is a multiple of 4 and every pointer and row start is 16-byte aligned (8 for bfloat16 rows).
template <typename TO, bool VEC>
__global__ void __launch_bounds__(LN_THREADS)
add_layernorm_kernel(float* __restrict__ h, LnAddends addends, const float* __restrict__ w1, const float* __restrict__ b1,
                     TO* __restrict__ out1, const float* __restrict__ w2, const float* __restrict__ b2, TO* __restrict__ out2,
                     const int* __restrict__ rows, int dim, float eps) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t t = rows ? (size_t)rows[r] : (size_t)r;
  float* hrow = h + t * dim;
  float sum = 0.f;
  if constexpr (VEC) {
    for (int e = 4 * threadIdx.x; e < dim; e += 4 * LN_THREADS) {
      float x[4];
      ln_load4(hrow, CWM_F32, e, x);
      for (int a = 0; a < addends.n; ++a) {
        const LnAddend& ad = addends.a[a];
        float y[4] = {0.f, 0.f, 0.f, 0.f};
        if (ad.n_partials == 1) {
          ln_load4(ad.ptr, ad.dtype, t * ad.ld + e, y);
        } else {
          // four partial sums in flight at a time, added in their order; what lies beyond the last is the last again, times zero
          for (int p = 0; p < ad.n_partials; p += 4) {
            float z[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) ln_load4(ad.ptr, ad.dtype, (size_t)min(p + u, ad.n_partials - 1) * ad.partial_stride + t * ad.ld + e, z[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const float keep = p + u < ad.n_partials ? 1.0f : 0.0f;
              y[0] = fmaf(keep, z[u][0], y[0]), y[1] = fmaf(keep, z[u][1], y[1]), y[2] = fmaf(keep, z[u][2], y[2]), y[3] = fmaf(keep, z[u][3], y[3]);
            }
          }
        }
        x[0] = fmaf(ad.scale, y[0], x[0]), x[1] = fmaf(ad.scale, y[1], x[1]);
        x[2] = fmaf(ad.scale, y[2], x[2]), x[3] = fmaf(ad.scale, y[3], x[3]);
      }
      if (!rows && addends.n > 0) *(float4*)(hrow + e) = make_float4(x[0], x[1], x[2], x[3]);
      *(float4*)(row + e) = make_float4(x[0], x[1], x[2], x[3]);
      sum += (x[0] + x[1]) + (x[2] + x[3]);
    }
  } else {
    for (int e = threadIdx.x; e < dim; e += LN_THREADS) {
      float x = hrow[e];
      for (int a = 0; a < addends.n; ++a) {
        const LnAddend& ad = addends.a[a];
        float y = 0.f;
        for (int p = 0; p < ad.n_partials; ++p) y += ln_load1(ad.ptr, ad.dtype, (size_t)p * ad.partial_stride + t * ad.ld + e);
        x = fmaf(ad.scale, y, x);
      }
      if (!rows && addends.n > 0) hrow[e] = x;
      row[e] = x;
      sum += x;
    }
  }
  if (!out1 && !out2) return;  // only the sum was wanted
  const float mean = block_sum(sum, scratch) / (float)dim;
  // every thread reads back what it wrote itself: no barrier is needed before this pass
  float sq = 0.f;
  if constexpr (VEC) {
    for (int e = 4 * threadIdx.x; e < dim; e += 4 * LN_THREADS) {
      const float4 x = *(const float4*)(row + e);
      const float d0 = x.x - mean, d1 = x.y - mean, d2 = x.z - mean, d3 = x.w - mean;
      sq += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
  } else {
    for (int e = threadIdx.x; e < dim; e += LN_THREADS) {
      const float d = row[e] - mean;
      sq += d * d;
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(sq, scratch) / (float)dim + eps);
  if constexpr (VEC) {
    for (int e = 4 * threadIdx.x; e < dim; e += 4 * LN_THREADS) {
      const float4 x = *(const float4*)(row + e);
      const float n[4] = {(x.x - mean) * rstd, (x.y - mean) * rstd, (x.z - mean) * rstd, (x.w - mean) * rstd};
      if (out1) {
        const float4 w = *(const float4*)(w1 + e), b = *(const float4*)(b1 + e);
        const float o[4] = {fmaf(n[0], w.x, b.x), fmaf(n[1], w.y, b.y), fmaf(n[2], w.z, b.z), fmaf(n[3], w.w, b.w)};
        LnStore<TO>::four(out1 + (size_t)r * dim + e, o);
      }
      if (out2) {
        const float4 w = *(const float4*)(w2 + e), b = *(const float4*)(b2 + e);
        const float o[4] = {fmaf(n[0], w.x, b.x), fmaf(n[1], w.y, b.y), fmaf(n[2], w.z, b.z), fmaf(n[3], w.w, b.w)};
        LnStore<TO>::four(out2 + (size_t)r * dim + e, o);
      }
    }
  } else {
    for (int e = threadIdx.x; e < dim; e += LN_THREADS) {
      const float n = (row[e] - mean) * rstd;
      if (out1) Elem<TO>::store(out1 + (size_t)r * dim + e, fmaf(n, w1[e], b1[e]));
      if (out2) Elem<TO>::store(out2 + (size_t)r * dim + e, fmaf(n, w2[e], b2[e]));
    }
  }
}

// h: float32 [T, dim], changed in place unless `rows` chooses rows.  Addend a: ptrs[a] of dtypes[a], rows lds[a]
// elements apart, n_partials[a] slabs partial_strides[a] elements apart, times scales[a].  w1, b1 (and w2, b2):
// float32 [dim]; out1 (and out2): [n_out, dim] of out_dtype, null for none (both null: only the sum is done).
extern "C" int cwm_add_layernorm(float* h, int n_addends, const void* const* ptrs, const int* dtypes, const long* lds,
                                 const int* n_partials, const long* partial_strides, const float* scales, const float* w1,
                                 const float* b1, void* out1, const float* w2, const float* b2, void* out2, int out_dtype,
                                 const int* rows, int n_out, int dim, float eps, hipStream_t stream) {
  CWM_REQUIRE(n_out >= 0 && dim >= 1 && dim <= LN_MAX_DIM, "add_layernorm: rows of %d elements are outside 1..%d", dim, LN_MAX_DIM);
  CWM_REQUIRE(n_addends >= 0 && n_addends <= LN_MAX_ADDENDS, "add_layernorm: %d addends, at most %d are taken", n_addends, LN_MAX_ADDENDS);
  CWM_REQUIRE(h, "add_layernorm: no residual");
  CWM_REQUIRE((!out1 || (w1 && b1)) && (!out2 || (w2 && b2)), "add_layernorm: a norm needs its weight and its bias");
  CWM_REQUIRE(eps > 0.f, "add_layernorm: eps must be positive");
  if (n_out == 0) return 0;
  LnAddends ad;
  ad.n = n_addends;
  bool vec = dim % 4 == 0 && ((uintptr_t)h % 16) == 0;
  for (int a = 0; a < n_addends; ++a) {
    CWM_REQUIRE(ptrs[a] && n_partials[a] >= 1, "add_layernorm: addend %d is empty", a);
    CWM_REQUIRE(n_partials[a] == 1 || dtypes[a] == CWM_F32, "add_layernorm: partial sums must be float32");
    ad.a[a] = LnAddend{ptrs[a], lds[a], partial_strides[a], n_partials[a], dtypes[a], scales[a]};
    const int bytes = dtypes[a] == CWM_F32 ? 4 : 2;
    vec = vec && lds[a] % 4 == 0 && partial_strides[a] % 4 == 0 && ((uintptr_t)ptrs[a] % (4 * bytes)) == 0;
  }
  const int out_bytes = out_dtype == CWM_F32 ? 4 : 2;
  vec = vec && ((uintptr_t)out1 % (4 * out_bytes)) == 0 && ((uintptr_t)out2 % (4 * out_bytes)) == 0;
  vec = vec && ((uintptr_t)w1 % 16) == 0 && ((uintptr_t)b1 % 16) == 0 && ((uintptr_t)w2 % 16) == 0 && ((uintptr_t)b2 % 16) == 0;
  const size_t lds_bytes = (size_t)dim * sizeof(float);
#define CWM_LN(TO, VEC)                                                                                                    \
  hipLaunchKernelGGL((add_layernorm_kernel<TO, VEC>), dim3(n_out), dim3(LN_THREADS), lds_bytes, stream, h, ad, w1, b1,       \
                     (TO*)out1, w2, b2, (TO*)out2, rows, dim, eps)
  if (out_dtype == CWM_F32) {
    if (vec) CWM_LN(float, true); else CWM_LN(float, false);
  } else if (out_dtype == CWM_BF16) {
    if (vec) CWM_LN(bf16_t, true); else CWM_LN(bf16_t, false);
  } else {
    return cwm_fail("add_layernorm: unknown output type %d", out_dtype);
  }
#undef CWM_LN
  return cwm_launch_status("add_layernorm");
}
