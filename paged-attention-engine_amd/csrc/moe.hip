// A feed-forward of many small gated experts, of which every token uses a few.
//
//   project_f32     float32 sums of a few output features (router logits, gate logits) from rows of either
//                   type: one wavefront an output, k shared out over its lanes in a fixed order
//   moe_route       per token: scores = softmax(logits) over all experts; the experts form `groups`
//                   equal groups of neighbours, a group's score is its largest score, only experts of the
//                   `keep` best groups can be chosen; the `top` largest scores among those are chosen,
//                   and their weights are the scores times `scale` (not renormalised).  Of equal
//                   scores the lower index wins.  One wavefront a token.
//   moe_gate_up     for every (token, chosen expert): act(W_gate x) * (W_up x), rounded to the activation type
//   moe_down        for every token: sum over its chosen experts of weight * W_down act, float32
//
// A token's routing and its experts' sums depend on that token alone, so its result does not depend on
// the batch.  The two expert kernels stream every chosen expert's weights once per (token, expert) pair;
// they are the kernels for steps of a few rows.
#include "common.h"
#include "api.h"

template <typename T>
__global__ __launch_bounds__(256) void project_f32_kernel(float* __restrict__ out, int64_t ldo, const T* __restrict__ A,
                                                          int64_t lda, const T* __restrict__ W,
                                                          const void* __restrict__ bias, int b_is_f32, int N, int K) {
  const int64_t t = blockIdx.x;
  const int n = blockIdx.y * 4 + threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  if (n >= N) return;
  const T* a = A + t * lda;
  const T* w = W + (int64_t)n * K;
  float sum = 0.f;
  for (int k = lane; k < K; k += PAE_WAVE) sum = fmaf(to_f32(a[k]), to_f32(w[k]), sum);
  sum = wave_sum(sum);
  if (lane == 0) out[t * ldo + n] = sum + (bias ? load_param(bias, b_is_f32, n) : 0.f);
}

extern "C" int pae_project_f32(int dtype, float* out, int64_t ldo, const void* A, int64_t lda, const void* W,
                               const void* bias, int b_is_f32, int M, int N, int K, hipStream_t stream) {
  PAE_REQUIRE(N > 0 && K > 0 && N <= 4 * 65535, "float32 projection: bad sizes N=%d K=%d", N, K);
  PAE_REQUIRE(ldo >= N && lda >= K, "float32 projection: row strides too small");
  if (M <= 0) return 0;
  dim3 grid(M, (N + 3) / 4);
  if (dtype == PAE_F32)
    project_f32_kernel<float><<<grid, 256, 0, stream>>>(out, ldo, (const float*)A, lda, (const float*)W, bias, b_is_f32, N, K);
  else if (dtype == PAE_BF16)
    project_f32_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, ldo, (const bf16_t*)A, lda, (const bf16_t*)W, bias, b_is_f32, N, K);
  else
    return pae_fail("float32 projection: unknown dtype code %d", dtype);
  return pae_check_launch("project_f32");
}

#define MOE_MAX_PER_LANE 16  // experts a lane holds: up to 1,024 experts

__global__ __launch_bounds__(PAE_WAVE) void moe_route_kernel(const float* __restrict__ logits, int E, int groups, int keep,
                                                             int top, float scale, int* __restrict__ chosen,
                                                             float* __restrict__ weights) {
  extern __shared__ float lds[];  // [E] scores, [groups] group scores
  float* score = lds;
  float* group_score = lds + E;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * E;
  float top_z = -INFINITY;
  for (int e = lane; e < E; e += PAE_WAVE) top_z = fmaxf(top_z, z[e]);
  top_z = wave_max(top_z);
  float sum = 0.f;
  for (int e = lane; e < E; e += PAE_WAVE) {
    const float p = expf(z[e] - top_z);
    score[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  __syncthreads();
  const int per_group = E / groups;
  for (int g = lane; g < groups; g += PAE_WAVE) {
    float best = -INFINITY;
    for (int j = 0; j < per_group; ++j) best = fmaxf(best, score[g * per_group + j]);
    group_score[g] = best;
  }
  __syncthreads();
  // an expert may be chosen if fewer than `keep` groups come before its own (a larger score, or an equal one
  // at a lower index)
  float mine[MOE_MAX_PER_LANE];
#pragma unroll
  for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
    const int e = lane + PAE_WAVE * j;
    mine[j] = -INFINITY;
    if (e < E) {
      const int g = e / per_group;
      const float gs = group_score[g];
      int before = 0;
      for (int o = 0; o < groups; ++o) before += (group_score[o] > gs || (group_score[o] == gs && o < g)) ? 1 : 0;
      if (before < keep) mine[j] = score[e];
    }
  }
  for (int r = 0; r < top; ++r) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
      if (mine[j] > best) {  // a lane's experts ascend with j: the first of equals stays
        best = mine[j];
        at = lane + PAE_WAVE * j;
      }
    for (int off = PAE_WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, PAE_WAVE);
      const int other_at = __shfl_xor(at, off, PAE_WAVE);
      if (other > best || (other == best && other_at < at)) {
        best = other;
        at = other_at;
      }
    }
    if (lane == 0) {
      chosen[t * top + r] = at;
      weights[t * top + r] = best / sum * scale;
    }
#pragma unroll
    for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
      if (lane + PAE_WAVE * j == at) mine[j] = -INFINITY;
  }
}

extern "C" int pae_moe_route(const float* logits, int num_tokens, int experts, int groups, int keep, int top, float scale,
                             int* chosen, float* weights, hipStream_t stream) {
  PAE_REQUIRE(experts > 0 && experts <= PAE_WAVE * MOE_MAX_PER_LANE, "routing: %d experts (1..%d)", experts,
              PAE_WAVE * MOE_MAX_PER_LANE);
  PAE_REQUIRE(groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups, "routing: %d groups of %d experts, %d kept",
              groups, experts, keep);
  PAE_REQUIRE(top > 0 && top <= keep * (experts / groups), "routing: %d experts chosen of %d that can be", top,
              keep * (experts / groups));
  if (num_tokens <= 0) return 0;
  moe_route_kernel<<<num_tokens, PAE_WAVE, (size_t)(experts + groups) * sizeof(float), stream>>>(
      logits, experts, groups, keep, top, scale, chosen, weights);
  return pae_check_launch("moe_route");
}

// One workgroup of four wavefronts per (pair, 16 features of the expert's width): a wavefront takes four
// features in turn, its lanes share out the hidden width.
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(T* __restrict__ act, const T* __restrict__ x, int64_t ldx,
                                                          const T* __restrict__ gate_w, const T* __restrict__ up_w,
                                                          const int* __restrict__ chosen, int top, int hidden, int inter,
                                                          int act_kind) {
  const int64_t pair = blockIdx.x;
  const int e = chosen[pair];
  const T* row = x + (pair / top) * ldx;
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  for (int j = 0; j < 4; ++j) {
    const int f = blockIdx.y * 16 + wave * 4 + j;
    if (f >= inter) return;
    const T* g = gate_w + ((int64_t)e * inter + f) * hidden;
    const T* u = up_w + ((int64_t)e * inter + f) * hidden;
    float gs = 0.f, us = 0.f;
    for (int k = lane; k < hidden; k += PAE_WAVE) {
      const float xv = to_f32(row[k]);
      gs = fmaf(xv, to_f32(g[k]), gs);
      us = fmaf(xv, to_f32(u[k]), us);
    }
    gs = wave_sum(gs);
    us = wave_sum(us);
    // both sums pass the activation type, as the products of the dense feed-forwards do
    if (lane == 0) act[pair * inter + f] = from_f32<T>(act_of(gs, act_kind) * us);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(float* __restrict__ out, const T* __restrict__ act,
                                                       const T* __restrict__ down_w, const int* __restrict__ chosen,
                                                       const float* __restrict__ weights, int top, int hidden, int inter) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  for (int j = 0; j < 4; ++j) {
    const int n = blockIdx.y * 16 + wave * 4 + j;
    if (n >= hidden) return;
    float total = 0.f;
    for (int r = 0; r < top; ++r) {
      const int e = chosen[t * top + r];
      const T* w = down_w + ((int64_t)e * hidden + n) * inter;
      const T* a = act + (t * top + r) * inter;
      float sum = 0.f;
      for (int k = lane; k < inter; k += PAE_WAVE) sum = fmaf(to_f32(a[k]), to_f32(w[k]), sum);
      total = fmaf(weights[t * top + r], wave_sum(sum), total);
    }
    if (lane == 0) out[t * hidden + n] = total;
  }
}

extern "C" int pae_moe_gate_up(int dtype, void* act, const void* x, int64_t ldx, const void* gate_w, const void* up_w,
                               const int* chosen, int num_tokens, int top, int hidden, int inter, int act_kind,
                               hipStream_t stream) {
  PAE_REQUIRE(top > 0 && hidden > 0 && inter > 0 && ldx >= hidden, "experts: bad sizes top=%d H=%d F=%d", top, hidden, inter);
  PAE_REQUIRE((inter + 15) / 16 <= 65535, "experts: width %d exceeds the grid", inter);
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens * top, (inter + 15) / 16);
  if (dtype == PAE_F32)
    moe_gate_up_kernel<float><<<grid, 256, 0, stream>>>((float*)act, (const float*)x, ldx, (const float*)gate_w,
                                                        (const float*)up_w, chosen, top, hidden, inter, act_kind);
  else if (dtype == PAE_BF16)
    moe_gate_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)x, ldx, (const bf16_t*)gate_w,
                                                         (const bf16_t*)up_w, chosen, top, hidden, inter, act_kind);
  else
    return pae_fail("experts: unknown dtype code %d", dtype);
  return pae_check_launch("moe_gate_up");
}

extern "C" int pae_moe_down(int dtype, float* out, const void* act, const void* down_w, const int* chosen,
                            const float* weights, int num_tokens, int top, int hidden, int inter, hipStream_t stream) {
  PAE_REQUIRE(top > 0 && hidden > 0 && inter > 0, "experts: bad sizes top=%d H=%d F=%d", top, hidden, inter);
  PAE_REQUIRE((hidden + 15) / 16 <= 65535, "experts: width %d exceeds the grid", hidden);
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens, (hidden + 15) / 16);
  if (dtype == PAE_F32)
    moe_down_kernel<float><<<grid, 256, 0, stream>>>(out, (const float*)act, (const float*)down_w, chosen, weights, top,
                                                     hidden, inter);
  else if (dtype == PAE_BF16)
    moe_down_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, (const bf16_t*)act, (const bf16_t*)down_w, chosen, weights, top,
                                                      hidden, inter);
  else
    return pae_fail("experts: unknown dtype code %d", dtype);
  return pae_check_launch("moe_down");
}
