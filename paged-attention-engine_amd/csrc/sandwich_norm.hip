// For blocks with a norm before and a norm after each sublayer: a sublayer's output joins the float32
// stream through the norm after it, and the new stream is handed on in the form its next reader wants.
//
//   y     = sum_j scale_j * term_j                      (float32, terms in the order given)
//   x    <- x + y / sqrt(mean(y^2) + eps) * w_out       (w_out absent: x <- x + y, no norm)
//   normed = x / sqrt(mean(x^2) + eps_next) * w_next    (optional: the norm before the next sublayer)
//   rows   = T(x)                                       (optional: the stream itself as a product's operand)
//
// A term is a sublayer's output [T, H] in the activation type, or float32 [T, H], or float32 partial sums
// [P, T, H] of a split product, which are added in order (two mixers side by side leave two terms with their
// factors, routed experts one term of as many parts as a token has experts).  One workgroup a row; the row
// waits in LDS between the passes, and a thread meets the same features in every pass.  Sums, both divisions
// and the stream are float32; a value is rounded once, when `normed` or `rows` is written.
#include "common.h"
#include "api.h"

#define PAE_JOIN_TERMS 4

struct JoinTerms {
  const void* ptr[PAE_JOIN_TERMS];
  int is_f32[PAE_JOIN_TERMS];
  int parts[PAE_JOIN_TERMS];
  int64_t part_stride[PAE_JOIN_TERMS];
  float scale[PAE_JOIN_TERMS];
  int count;
};

template <typename T>
__device__ __forceinline__ void join_load4(const T* p, float (&v)[4]);
template <>
__device__ __forceinline__ void join_load4<float>(const float* p, float (&v)[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <>
__device__ __forceinline__ void join_load4<bf16_t>(const bf16_t* p, float (&v)[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);  // a bfloat16 is the upper half of a float
  v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
  v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
}

template <typename T>
__device__ __forceinline__ void join_store4(T* p, const float (&v)[4]);
template <>
__device__ __forceinline__ void join_store4<float>(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
__device__ __forceinline__ void join_store4<bf16_t>(bf16_t* p, const float (&v)[4]) {
  bf16_t h[4] = {__float2bfloat16(v[0]), __float2bfloat16(v[1]), __float2bfloat16(v[2]), __float2bfloat16(v[3])};
  *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(h);
}

// VEC: four consecutive features a thread and trip (widths in multiples of four), else one.  The first pass only
// reads (the terms and, ahead of its use, the stream), so that all of a trip's loads are in flight together.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void norm_join_kernel(float* __restrict__ residual, JoinTerms terms,
                                                        const void* __restrict__ w_out, int w_out_is_f32, float eps,
                                                        const void* __restrict__ w_next, int w_next_is_f32,
                                                        float eps_next, T* __restrict__ normed, T* __restrict__ rows,
                                                        int hidden) {
  extern __shared__ float row_lds[];  // [2][hidden]: the sublayer's row, then the stream's
  __shared__ float scratch[4];
  constexpr int W = VEC ? 4 : 1;
  float* y_lds = row_lds;
  float* x_lds = row_lds + hidden;
  const int64_t base = (int64_t)blockIdx.x * hidden;
  float* x = residual + base;
  float ss = 0.f;
  for (int i = threadIdx.x * W; i < hidden; i += 256 * W) {
    float xv[4] = {0.f, 0.f, 0.f, 0.f}, y[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) join_load4<float>(x + i, xv);
    else xv[0] = x[i];
    // (constant indices: a run-time index would move the terms' description into private memory)
#pragma unroll
    for (int j = 0; j < PAE_JOIN_TERMS; ++j) {
      if (j >= terms.count) break;
      float sum[4] = {0.f, 0.f, 0.f, 0.f};
      if (terms.is_f32[j]) {
        const float* p = (const float*)terms.ptr[j] + base + i;
        for (int part = 0; part < terms.parts[j]; ++part) {
          float t[4] = {0.f, 0.f, 0.f, 0.f};
          if (VEC) join_load4<float>(p + part * terms.part_stride[j], t);
          else t[0] = p[part * terms.part_stride[j]];
#pragma unroll
          for (int e = 0; e < W; ++e) sum[e] += t[e];
        }
      } else {
        const T* p = (const T*)terms.ptr[j] + base + i;
        if (VEC) join_load4<T>(p, sum);
        else sum[0] = to_f32(p[0]);
      }
#pragma unroll
      for (int e = 0; e < W; ++e) y[e] += terms.scale[j] * sum[e];
    }
#pragma unroll
    for (int e = 0; e < W; ++e) {
      y_lds[i + e] = y[e];
      x_lds[i + e] = xv[e];
      ss = fmaf(y[e], y[e], ss);
    }
  }
  float inv = 1.f;
  if (w_out) {
    ss = block_sum<4>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  }
  float sx = 0.f;
  for (int i = threadIdx.x * W; i < hidden; i += 256 * W) {
    float v[4];
#pragma unroll
    for (int e = 0; e < W; ++e) {
      const float branch = w_out ? y_lds[i + e] * inv * load_param(w_out, w_out_is_f32, i + e) : y_lds[i + e];
      v[e] = x_lds[i + e] + branch;
      x_lds[i + e] = v[e];
      sx = fmaf(v[e], v[e], sx);
    }
    if (VEC) {
      join_store4<float>(x + i, v);
      if (rows) join_store4<T>(rows + base + i, v);
    } else {
      x[i] = v[0];
      if (rows) rows[base + i] = from_f32<T>(v[0]);
    }
  }
  if (!normed) return;
  sx = block_sum<4>(sx, scratch);
  const float inv_next = 1.0f / sqrtf(sx / (float)hidden + eps_next);
  for (int i = threadIdx.x * W; i < hidden; i += 256 * W) {
    float v[4];
#pragma unroll
    for (int e = 0; e < W; ++e) v[e] = x_lds[i + e] * inv_next * load_param(w_next, w_next_is_f32, i + e);
    if (VEC) join_store4<T>(normed + base + i, v);
    else normed[base + i] = from_f32<T>(v[0]);
  }
}

extern "C" int pae_norm_join(int dtype, float* residual, int num_terms, const void* const* term_ptr, const int* term_is_f32,
                             const int* term_parts, const int64_t* term_part_stride, const float* term_scale,
                             const void* w_out, int w_out_is_f32, float eps, const void* w_next, int w_next_is_f32,
                             float eps_next, void* normed, void* rows, int num_rows, int hidden, hipStream_t stream) {
  PAE_REQUIRE(num_terms >= 0 && num_terms <= PAE_JOIN_TERMS, "norm and join: %d terms (at most %d)", num_terms, PAE_JOIN_TERMS);
  PAE_REQUIRE(hidden > 0 && hidden <= 7680, "norm and join: width %d is outside 1..7680", hidden);
  PAE_REQUIRE(!normed || w_next, "norm and join: the next norm's rows are asked for without its weight");
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "norm and join: unknown dtype code %d", dtype);
  if (num_rows <= 0) return 0;
  JoinTerms terms;
  terms.count = num_terms;
  for (int j = 0; j < PAE_JOIN_TERMS; ++j) {
    terms.ptr[j] = nullptr;
    terms.is_f32[j] = 0;
    terms.parts[j] = 1;
    terms.part_stride[j] = 0;
    terms.scale[j] = 0.f;
  }
  for (int j = 0; j < num_terms; ++j) {
    PAE_REQUIRE(term_ptr[j] && term_parts[j] >= 1 && (term_is_f32[j] || term_parts[j] == 1), "norm and join: bad term %d", j);
    terms.ptr[j] = term_ptr[j];
    terms.is_f32[j] = term_is_f32[j];
    terms.parts[j] = term_parts[j];
    terms.part_stride[j] = term_part_stride[j];
    terms.scale[j] = term_scale[j];
  }
  const size_t lds = 2 * (size_t)hidden * sizeof(float);
  bool vec = hidden % 4 == 0 && (uintptr_t)residual % 16 == 0 && (uintptr_t)normed % 16 == 0 && (uintptr_t)rows % 16 == 0;
  for (int j = 0; j < num_terms; ++j) vec = vec && (uintptr_t)term_ptr[j] % 16 == 0 && term_part_stride[j] % 4 == 0;
#define NORM_JOIN(T, VEC)                                                                                           \
  norm_join_kernel<T, VEC><<<num_rows, 256, lds, stream>>>(residual, terms, w_out, w_out_is_f32, eps, w_next,        \
                                                           w_next_is_f32, eps_next, (T*)normed, (T*)rows, hidden)
  if (dtype == PAE_F32) {
    if (vec) NORM_JOIN(float, true);
    else NORM_JOIN(float, false);
  } else {
    if (vec) NORM_JOIN(bf16_t, true);
    else NORM_JOIN(bf16_t, false);
  }
#undef NORM_JOIN
  return pae_check_launch("norm_join");
}
