// For blocks whose branches all read the same stream: the branches of the block before join the
// float32 residual, and the new residual is normed twice, once for each branch of this block.
//
//   x <- x + sum_j scale_j * term_j          (float32, terms in the order given)
//   out1 = x / sqrt(mean(x^2) + eps) * w1,   out2 = the same with w2
//
// A term is a branch's output [T, H] in the activation type, or float32 [T, H], or float32 partial
// sums [P, T, H] of a split product, which are added in order.  Either output may be absent; with
// `rows` only those rows are produced and nothing is written back.  One workgroup a row; the row
// waits in LDS between the two passes.
#include "common.h"
#include "api.h"

#define PAE_MAX_TERMS 4

struct SumTerms {
  const void* ptr[PAE_MAX_TERMS];
  int is_f32[PAE_MAX_TERMS];
  int parts[PAE_MAX_TERMS];
  int64_t part_stride[PAE_MAX_TERMS];
  float scale[PAE_MAX_TERMS];
  int count;
};

template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&v)[4]);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <>
__device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float (&v)[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);  // a bfloat16 is the upper half of a float
  v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
  v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
}

// VEC: four consecutive features a thread and trip (widths in multiples of four), else one.  The first pass only
// reads memory (the new row goes to LDS), so that nothing keeps its loads from being in flight together; the
// second writes the stream and the norms.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sum_norm2_kernel(float* __restrict__ residual, SumTerms terms,
                                                        const void* __restrict__ w1, int w1_is_f32,
                                                        const void* __restrict__ w2, int w2_is_f32, float eps,
                                                        const int* __restrict__ rows, T* __restrict__ out1,
                                                        T* __restrict__ out2, int hidden, int write_residual) {
  extern __shared__ float row_lds[];  // [hidden]
  __shared__ float scratch[4];
  constexpr int W = VEC ? 4 : 1;
  const int64_t src = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = residual + src * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x * W; i < hidden; i += 256 * W) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) load4<float>(x + i, v);
    else v[0] = x[i];
    // (the terms are walked with constant indices: an index that is only known at run time would move the
    // whole description from the kernel's arguments into private memory)
#pragma unroll
    for (int j = 0; j < PAE_MAX_TERMS; ++j) {
      if (j >= terms.count) break;
      float sum[4] = {0.f, 0.f, 0.f, 0.f};
      if (terms.is_f32[j]) {
        const float* p = (const float*)terms.ptr[j] + src * hidden + i;
        for (int part = 0; part < terms.parts[j]; ++part) {
          float t[4] = {0.f, 0.f, 0.f, 0.f};
          if (VEC) load4<float>(p + part * terms.part_stride[j], t);
          else t[0] = p[part * terms.part_stride[j]];
#pragma unroll
          for (int e = 0; e < W; ++e) sum[e] += t[e];
        }
      } else {
        const T* p = (const T*)terms.ptr[j] + src * hidden + i;
        if (VEC) load4<T>(p, sum);
        else sum[0] = to_f32(p[0]);
      }
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] += terms.scale[j] * sum[e];
    }
#pragma unroll
    for (int e = 0; e < W; ++e) {
      row_lds[i + e] = v[e];
      ss = fmaf(v[e], v[e], ss);
    }
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  const int64_t dst = (int64_t)blockIdx.x * hidden;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float v = row_lds[i];
    if (write_residual) x[i] = v;
    const float n = v * inv;
    if (out1) out1[dst + i] = from_f32<T>(n * load_param(w1, w1_is_f32, i));
    if (out2) out2[dst + i] = from_f32<T>(n * load_param(w2, w2_is_f32, i));
  }
}

extern "C" int pae_sum_norm2(int dtype, float* residual, int num_terms, const void* const* term_ptr, const int* term_is_f32,
                             const int* term_parts, const int64_t* term_part_stride, const float* term_scale,
                             const void* w1, int w1_is_f32, const void* w2, int w2_is_f32, float eps, const int* rows,
                             void* out1, void* out2, int num_rows, int hidden, int write_residual, hipStream_t stream) {
  PAE_REQUIRE(num_terms >= 0 && num_terms <= PAE_MAX_TERMS, "sum and norms: %d terms (at most %d)", num_terms, PAE_MAX_TERMS);
  PAE_REQUIRE(hidden > 0 && hidden <= 15360, "sum and norms: width %d is outside 1..15360", hidden);
  PAE_REQUIRE((!out1 || w1) && (!out2 || w2), "sum and norms: an output without its weight");
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "sum and norms: unknown dtype code %d", dtype);
  if (num_rows <= 0) return 0;
  SumTerms terms;
  terms.count = num_terms;
  for (int j = 0; j < num_terms; ++j) {
    PAE_REQUIRE(term_ptr[j] && term_parts[j] >= 1 && (term_is_f32[j] || term_parts[j] == 1), "sum and norms: bad term %d", j);
    terms.ptr[j] = term_ptr[j];
    terms.is_f32[j] = term_is_f32[j];
    terms.parts[j] = term_parts[j];
    terms.part_stride[j] = term_part_stride[j];
    terms.scale[j] = term_scale[j];
  }
  const size_t lds = (size_t)hidden * sizeof(float);
  bool vec = hidden % 4 == 0 && (uintptr_t)residual % 16 == 0;
  for (int j = 0; j < num_terms; ++j) vec = vec && (uintptr_t)term_ptr[j] % 16 == 0 && term_part_stride[j] % 4 == 0;
#define SUM_NORM2(T, VEC)                                                                                          \
  sum_norm2_kernel<T, VEC><<<num_rows, 256, lds, stream>>>(residual, terms, w1, w1_is_f32, w2, w2_is_f32, eps, rows, \
                                                           (T*)out1, (T*)out2, hidden, rows ? 0 : write_residual)
  if (dtype == PAE_F32) {
    if (vec) SUM_NORM2(float, true);
    else SUM_NORM2(float, false);
  } else {
    if (vec) SUM_NORM2(bf16_t, true);
    else SUM_NORM2(bf16_t, false);
  }
#undef SUM_NORM2
  return pae_check_launch("sum_norm2");
}
