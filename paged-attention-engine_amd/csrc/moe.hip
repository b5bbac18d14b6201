// A feed-forward of many small gated experts, of which every token uses a few.
//
//   project_f32     float32 sums of a few output features (router logits, gate logits) from rows of either
//                   type: one wavefront an output, k shared out over its lanes in a fixed order
//   moe_route       per token: scores = softmax(logits) over all experts; the experts form `groups`
//                   equal groups of neighbours, a group's score is its largest score, only experts of the
//                   `keep` best groups can be chosen; the `top` largest scores among those are chosen,
//                   and their weights are the scores times `scale` (not renormalised).  Of equal
//                   scores the lower index wins.  With a `choice_bias` [E], experts and groups are compared
//                   by score + bias, while the weights stay the scores themselves.  One wavefront a token.
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

// The same sums with 16-byte loads, for rows and widths that allow them: a workgroup takes one row and `per_wave`
// outputs for each of its four wavefronts (all of a row's outputs in steps of many rows, one each in steps of
// few); a lane adds its 8 (or 4) consecutive k of every 64-lane stretch, then the lanes meet.
template <typename T>
__global__ __launch_bounds__(256) void project_f32_wide_kernel(float* __restrict__ out, int64_t ldo, const T* __restrict__ A,
                                                               int64_t lda, const T* __restrict__ W,
                                                               const void* __restrict__ bias, int b_is_f32, int N, int K,
                                                               int per_wave) {
  constexpr int VEC = 16 / sizeof(T);
  struct alignas(16) Chunk { T v[VEC]; };
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  const T* a = A + t * lda;
  const int first = blockIdx.y * 4 * per_wave + wave;
  for (int n = first; n < N && n < first + 4 * per_wave; n += 4) {
    const T* w = W + (int64_t)n * K;
    float sum = 0.f;
    for (int k = lane * VEC; k < K; k += PAE_WAVE * VEC) {
      const Chunk x = *reinterpret_cast<const Chunk*>(a + k);
      const Chunk y = *reinterpret_cast<const Chunk*>(w + k);
#pragma unroll
      for (int i = 0; i < VEC; ++i) sum = fmaf(to_f32(x.v[i]), to_f32(y.v[i]), sum);
    }
    sum = wave_sum(sum);
    if (lane == 0) out[t * ldo + n] = sum + (bias ? load_param(bias, b_is_f32, n) : 0.f);
  }
}

extern "C" int pae_project_f32(int dtype, float* out, int64_t ldo, const void* A, int64_t lda, const void* W,
                               const void* bias, int b_is_f32, int M, int N, int K, hipStream_t stream) {
  PAE_REQUIRE(N > 0 && K > 0 && N <= 4 * 65535, "float32 projection: bad sizes N=%d K=%d", N, K);
  PAE_REQUIRE(ldo >= N && lda >= K, "float32 projection: row strides too small");
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "float32 projection: unknown dtype code %d", dtype);
  if (M <= 0) return 0;
  const int vec = dtype == PAE_F32 ? 4 : 8;
  const bool wide = K % vec == 0 && lda % vec == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0;
  dim3 grid(M, (N + 3) / 4);
  const int per_wave = M >= 512 ? (N + 3) / 4 : 1;
  dim3 wide_grid(M, (N + 4 * per_wave - 1) / (4 * per_wave));
  if (dtype == PAE_F32) {
    if (wide)
      project_f32_wide_kernel<float><<<wide_grid, 256, 0, stream>>>(out, ldo, (const float*)A, lda, (const float*)W, bias, b_is_f32, N, K, per_wave);
    else
      project_f32_kernel<float><<<grid, 256, 0, stream>>>(out, ldo, (const float*)A, lda, (const float*)W, bias, b_is_f32, N, K);
  } else {
    if (wide)
      project_f32_wide_kernel<bf16_t><<<wide_grid, 256, 0, stream>>>(out, ldo, (const bf16_t*)A, lda, (const bf16_t*)W, bias, b_is_f32, N, K, per_wave);
    else
      project_f32_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, ldo, (const bf16_t*)A, lda, (const bf16_t*)W, bias, b_is_f32, N, K);
  }
  return pae_check_launch("project_f32");
}

#define MOE_MAX_PER_LANE 16  // experts a lane holds: up to 1,024 experts

__global__ __launch_bounds__(PAE_WAVE) void moe_route_kernel(const float* __restrict__ logits, int E, int groups, int keep,
                                                             int top, float scale, const float* __restrict__ choice_bias,
                                                             int* __restrict__ chosen, float* __restrict__ weights) {
  extern __shared__ float lds[];  // [E] scores, [groups] group scores, and with a bias [E] what experts are compared by
  float* score = lds;
  float* group_score = lds + E;
  float* rank = choice_bias ? group_score + groups : score;
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
  if (choice_bias)
    for (int e = lane; e < E; e += PAE_WAVE) rank[e] = score[e] / sum + choice_bias[e];
  __syncthreads();
  const int per_group = E / groups;
  for (int g = lane; g < groups; g += PAE_WAVE) {
    float best = -INFINITY;
    for (int j = 0; j < per_group; ++j) best = fmaxf(best, rank[g * per_group + j]);
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
      if (before < keep) mine[j] = rank[e];
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
      weights[t * top + r] = score[at] / sum * scale;
    }
#pragma unroll
    for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
      if (lane + PAE_WAVE * j == at) mine[j] = -INFINITY;
  }
}

extern "C" int pae_moe_route(const float* logits, int num_tokens, int experts, int groups, int keep, int top, float scale,
                             const float* choice_bias, int* chosen, float* weights, hipStream_t stream) {
  PAE_REQUIRE(experts > 0 && experts <= PAE_WAVE * MOE_MAX_PER_LANE, "routing: %d experts (1..%d)", experts,
              PAE_WAVE * MOE_MAX_PER_LANE);
  PAE_REQUIRE(groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups, "routing: %d groups of %d experts, %d kept",
              groups, experts, keep);
  PAE_REQUIRE(top > 0 && top <= keep * (experts / groups), "routing: %d experts chosen of %d that can be", top,
              keep * (experts / groups));
  if (num_tokens <= 0) return 0;
  moe_route_kernel<<<num_tokens, PAE_WAVE, (size_t)(experts + groups + (choice_bias ? experts : 0)) * sizeof(float), stream>>>(
      logits, experts, groups, keep, top, scale, choice_bias, chosen, weights);
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
    // the gate is applied to the float32 sums and the product rounded once
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

// ---------------------------------------------------------------------------------------------------------------
// The experts on the matrix cores (bfloat16, widths in multiples of 32).  The (token, expert) pairs of a step are
// sorted by expert on the device, and every expert's pairs are cut into tiles of up to 16 MT rows; a workgroup takes one
// tile and 64 or more output features, its four wavefronts a quarter each, so an expert's weights are streamed once per
// tile: once in all for a step of a few tokens, and once per 16 MT of an expert's tokens in a prompt.  Which tile a
// pair falls into changes nothing of its sums (k ascends in steps of 32 for every row by itself), so a token's
// result does not depend on the batch.
//
//   moe_sort            counts, offsets and tiles by expert (one workgroup; the order of an expert's pairs among
//                       themselves is whatever the counters' turn gives, and does not matter)
//   gate/up             act(W_gate x) * (W_up x) for a tile's rows, rounded, to rows in sorted order
//   down                weight * W_down act for a tile's rows, float32, to y[chosen place][token]: the `top` places
//                       of a token are float32 partial sums that the stream's next norm adds in order
// each in three kernels by the step's size: moe_few_tiles (up to 512 pairs), moe_tiles_gate_up / moe_tiles_down (up to
// 4,096), moe_big_tiles (above).
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ chosen, int pairs, int experts, int tile_rows,
                                                        int* __restrict__ order, int4* __restrict__ tiles, int max_tiles) {
  extern __shared__ int sorted_lds[];  // [experts] counts, starts, cursors, first tiles; [1] tiles in all
  int* count = sorted_lds;
  int* start = count + experts;
  int* cursor = start + experts;
  int* first_tile = cursor + experts;
  int* total = first_tile + experts;
  for (int e = threadIdx.x; e < experts; e += 1024) count[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += 1024) atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int rows = 0, tile = 0;
    for (int e = 0; e < experts; ++e) {
      start[e] = rows;
      first_tile[e] = tile;
      rows += count[e];
      tile += (count[e] + tile_rows - 1) / tile_rows;
    }
    *total = tile;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += 1024) {
    const int e = chosen[p];
    order[start[e] + atomicAdd(&cursor[e], 1)] = p;
  }
  for (int e = threadIdx.x; e < experts; e += 1024)
    for (int j = 0; j * tile_rows < count[e]; ++j)
      tiles[first_tile[e] + j] = make_int4(e, start[e] + j * tile_rows, min(tile_rows, count[e] - j * tile_rows), 0);
  for (int i = *total + threadIdx.x; i < max_tiles; i += 1024) tiles[i] = make_int4(0, 0, 0, 0);
}

// A wavefront holds MT tiles of 16 rows by NT tiles of 16 features: MT + NT (2 NT with gate and up) operand loads
// feed MT NT (2 MT NT) matrix instructions in every step of 32 of k.
template <int MT, int NT>
__global__ __launch_bounds__(256) void moe_tiles_gate_up_kernel(bf16_t* __restrict__ act, const bf16_t* __restrict__ x,
                                                                int64_t ldx, const bf16_t* __restrict__ gate_w,
                                                                const bf16_t* __restrict__ up_w, const int* __restrict__ order,
                                                                const int4* __restrict__ tiles, int top, int hidden, int inter,
                                                                int act_kind) {
  const int4 tile = tiles[blockIdx.x];  // (expert, first sorted row, rows, unused)
  const int lane = threadIdx.x % PAE_WAVE, wave = threadIdx.x / PAE_WAVE;
  const int col = lane % 16, kg = lane / 16;
  const int f0 = (blockIdx.y * 4 + wave) * 16 * NT;
  if (tile.z <= 0 || f0 >= inter) return;
  const bf16_t* gw[NT];
  const bf16_t* uw[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int64_t w_row = (int64_t)tile.x * inter + min(f0 + 16 * nt + col, inter - 1);
    gw[nt] = gate_w + w_row * hidden + 8 * kg;
    uw[nt] = up_w + w_row * hidden + 8 * kg;
  }
  const bf16_t* rows[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + col;
    rows[mt] = x + (int64_t)(order[tile.y + (r < tile.z ? r : 0)] / top) * ldx + 8 * kg;
  }
  f32x4 gs[MT][NT], us[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) gs[mt][nt] = us[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // operands of the step after are on their way while a step's matrix instructions run; the loop's loads are
  // unconditional and the last step stands by itself
  bf16x8 g[2][NT], u[2][NT], a[2][MT];
  auto load = [&](int set, int k) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      g[set][nt] = *reinterpret_cast<const bf16x8*>(gw[nt] + k);
      u[set][nt] = *reinterpret_cast<const bf16x8*>(uw[nt] + k);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a[set][mt] = *reinterpret_cast<const bf16x8*>(rows[mt] + k);
  };
  auto multiply = [&](int set) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        gs[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g[set][nt], a[set][mt], gs[mt][nt], 0, 0, 0);
        us[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u[set][nt], a[set][mt], us[mt][nt], 0, 0, 0);
      }
  };
  load(0, 0);
  int k = 0;
  for (; k + 64 < hidden; k += 64) {
    load(1, k + 32);
    multiply(0);
    load(0, k + 64);
    multiply(1);
  }
  if (k + 32 < hidden) {
    load(1, k + 32);
    multiply(0);
    multiply(1);
  } else {
    multiply(0);
  }
  // a lane holds features f0 + 16 nt + 4 kg .. + 3 of the row mt * 16 + col
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + col;
    if (r >= tile.z) continue;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int f = f0 + 16 * nt + 4 * kg;
      bf16_t* o = act + (int64_t)(tile.y + r) * inter + f;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (f + i < inter) o[i] = __float2bfloat16(act_of(gs[mt][nt][i], act_kind) * us[mt][nt][i]);
    }
  }
}

template <int MT, int NT>
__global__ __launch_bounds__(256) void moe_tiles_down_kernel(float* __restrict__ y, const bf16_t* __restrict__ act,
                                                             const bf16_t* __restrict__ down_w, const int* __restrict__ order,
                                                             const float* __restrict__ weights, const int4* __restrict__ tiles,
                                                             int top, int num_tokens, int hidden, int inter) {
  const int4 tile = tiles[blockIdx.x];
  const int lane = threadIdx.x % PAE_WAVE, wave = threadIdx.x / PAE_WAVE;
  const int col = lane % 16, kg = lane / 16;
  const int n0 = (blockIdx.y * 4 + wave) * 16 * NT;
  if (tile.z <= 0 || n0 >= hidden) return;
  const bf16_t* w[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    w[nt] = down_w + ((int64_t)tile.x * hidden + min(n0 + 16 * nt + col, hidden - 1)) * inter + 8 * kg;
  const bf16_t* rows[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + col;
    rows[mt] = act + (int64_t)(tile.y + (r < tile.z ? r : 0)) * inter + 8 * kg;
  }
  f32x4 sums[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) sums[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wk[2][NT], a[2][MT];
  auto load = [&](int set, int k) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wk[set][nt] = *reinterpret_cast<const bf16x8*>(w[nt] + k);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a[set][mt] = *reinterpret_cast<const bf16x8*>(rows[mt] + k);
  };
  auto multiply = [&](int set) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        sums[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wk[set][nt], a[set][mt], sums[mt][nt], 0, 0, 0);
  };
  load(0, 0);
  int k = 0;
  for (; k + 64 < inter; k += 64) {
    load(1, k + 32);
    multiply(0);
    load(0, k + 64);
    multiply(1);
  }
  if (k + 32 < inter) {
    load(1, k + 32);
    multiply(0);
    multiply(1);
  } else {
    multiply(0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + col;
    if (r >= tile.z) continue;
    const int pair = order[tile.y + r];
    const float weight = weights[pair];
    float* row = y + ((int64_t)(pair % top) * num_tokens + pair / top) * hidden;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int n = n0 + 16 * nt + 4 * kg;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < hidden) row[n + i] = weight * sums[mt][nt][i];
    }
  }
}

// The two products for steps of up to 512 pairs (decode steps, small portions), where an expert sees at most a few
// tokens and its weights are streamed exactly once: a tile is up to 16 rows, and the four wavefronts of a workgroup share
// one tile of 16 features and take a quarter of k each, leave their sums in LDS, and the first adds them in wavefront
// order (a wavefront per 16 features and the whole of k was measured against it: 35 + 22 us against 25 + 14 at one
// token, 85 + 57 against 67 + 39 at eight).  The order of adding is a function of the sizes alone.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_few_tiles_kernel(bf16_t* __restrict__ act_out, float* __restrict__ y,
                                                            const bf16_t* __restrict__ a_rows, int64_t lda,
                                                            const bf16_t* __restrict__ w_first, const bf16_t* __restrict__ w_second,
                                                            const int* __restrict__ order, const float* __restrict__ weights,
                                                            const int4* __restrict__ tiles, int top, int num_tokens, int K,
                                                            int N, int act_kind) {
  __shared__ f32x4 parts[3][2][PAE_WAVE];
  const int4 tile = tiles[blockIdx.x];  // (expert, first sorted row, rows <= 16, unused)
  const int lane = threadIdx.x % PAE_WAVE, wave = threadIdx.x / PAE_WAVE;
  const int col = lane % 16, kg = lane / 16;
  const int n0 = blockIdx.y * 16;
  if (tile.z <= 0 || n0 >= N) return;
  const int64_t w_row = (int64_t)tile.x * N + min(n0 + col, N - 1);
  const bf16_t* w1 = w_first + w_row * K + 8 * kg;
  const bf16_t* w2 = GATED ? w_second + w_row * K + 8 * kg : nullptr;
  const int sorted = tile.y + (col < tile.z ? col : 0);
  const bf16_t* a = a_rows + (int64_t)(GATED ? order[sorted] / top : sorted) * lda + 8 * kg;
  const int steps = K / 32, per = (steps + 3) / 4;
  const int first = wave * per, last = min(steps, first + per);
  f32x4 s1 = {0.f, 0.f, 0.f, 0.f}, s2 = {0.f, 0.f, 0.f, 0.f};
  if (first < last) {
    bf16x8 ca = *reinterpret_cast<const bf16x8*>(a + 32 * first), c1 = *reinterpret_cast<const bf16x8*>(w1 + 32 * first), c2;
    if (GATED) c2 = *reinterpret_cast<const bf16x8*>(w2 + 32 * first);
    for (int st = first + 1; st < last; ++st) {
      const bf16x8 na = *reinterpret_cast<const bf16x8*>(a + 32 * st), n1 = *reinterpret_cast<const bf16x8*>(w1 + 32 * st);
      bf16x8 n2;
      if (GATED) n2 = *reinterpret_cast<const bf16x8*>(w2 + 32 * st);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c1, ca, s1, 0, 0, 0);
      if (GATED) s2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c2, ca, s2, 0, 0, 0);
      ca = na; c1 = n1;
      if (GATED) c2 = n2;
    }
    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c1, ca, s1, 0, 0, 0);
    if (GATED) s2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c2, ca, s2, 0, 0, 0);
  }
  if (wave > 0) {
    parts[wave - 1][0][lane] = s1;
    if (GATED) parts[wave - 1][1][lane] = s2;
  }
  __syncthreads();
  if (wave > 0 || col >= tile.z) return;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    s1 += parts[w][0][lane];
    if (GATED) s2 += parts[w][1][lane];
  }
  const int n = n0 + 4 * kg;  // a lane holds features n .. n + 3 of the row col
  if (GATED) {
    bf16_t* o = act_out + (int64_t)(tile.y + col) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) o[i] = __float2bfloat16(act_of(s1[i], act_kind) * s2[i]);
  } else {
    const int pair = order[tile.y + col];
    const float weight = weights[pair];
    float* o = y + ((int64_t)(pair % top) * num_tokens + pair / top) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) o[i] = weight * s1[i];
  }
}

// The same two products for prompts, where an expert sees hundreds of tokens: a workgroup takes a tile of 128 rows
// and 128 features with gate and up (or 256 output features of the down product), and its operands pass through LDS:
// every 64 of k, the 256 threads fetch 128 rows of activations and 256 rows of weights, a whole 128-byte line a row, into
// registers while the step before is multiplied, and then write them to LDS (rows 144 bytes apart, so that the 16-byte
// reads of a wavefront's lanes fall on all banks).  The four wavefronts are two by two: 64 rows by 64 features with gate
// and up (or 128 features), 64 matrix instructions for 24 reads of LDS a step.  Two barriers a step.
#define MOE_BIG_ROWS 128
#define MOE_BIG_K 64
#define MOE_LDS_STRIDE 72  // bf16 from a row of 64 to the next in LDS
template <bool GATED>
__global__ __launch_bounds__(256) void moe_big_tiles_kernel(bf16_t* __restrict__ act_out, float* __restrict__ y,
                                                            const bf16_t* __restrict__ a_rows, int64_t lda,
                                                            const bf16_t* __restrict__ w_first, const bf16_t* __restrict__ w_second,
                                                            const int* __restrict__ order, const float* __restrict__ weights,
                                                            const int4* __restrict__ tiles, int top, int num_tokens, int K,
                                                            int N, int act_kind) {
  // GATED: a_rows = x (row of a pair = its token), w_first / w_second = gate / up [E][N][K], N = the experts' width;
  // else: a_rows = act in sorted order, w_first = down [E][N][K], N = the hidden width
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[MOE_BIG_ROWS * MOE_LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t lds_w[256 * MOE_LDS_STRIDE];
  const int4 tile = tiles[blockIdx.x];  // (expert, first sorted row, rows, unused)
  if (tile.z <= 0) return;
  constexpr int FEATURES = GATED ? 128 : 256;  // output features a workgroup takes
  const int n_base = blockIdx.y * FEATURES;
  const int tid = threadIdx.x, lane = tid % PAE_WAVE, wave = tid / PAE_WAVE;
  const int col = lane % 16, kg = lane / 16;
  const int wr = wave / 2, wc = wave % 2;
  // what this thread fetches: 16 bytes (piece tid % 8) of rows tid / 8 + 32 j
  const int piece = tid % 8, frow = tid / 8;
  const bf16_t* a_src[4];
  const bf16_t* w_src[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = frow + 32 * j;
    const int sorted = tile.y + (r < tile.z ? r : 0);
    const int64_t row = GATED ? order[sorted] / top : sorted;
    a_src[j] = a_rows + row * lda + 8 * piece;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int r = frow + 32 * j;  // row of the 256 in LDS: gated, the first 128 are gate's features, the rest up's
    const int n = min(n_base + (GATED ? r % 128 : r), N - 1);
    const bf16_t* w = (GATED && r >= 128) ? w_second : w_first;
    w_src[j] = w + ((int64_t)tile.x * N + n) * K + 8 * piece;
  }
  f32x4 acc[4][8];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 fa[4], fw[8];
  auto fetch = [&](int k) {
#pragma unroll
    for (int j = 0; j < 4; ++j) fa[j] = *reinterpret_cast<const bf16x8*>(a_src[j] + k);
#pragma unroll
    for (int j = 0; j < 8; ++j) fw[j] = *reinterpret_cast<const bf16x8*>(w_src[j] + k);
  };
  auto stage = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<bf16x8*>(&lds_a[(frow + 32 * j) * MOE_LDS_STRIDE + 8 * piece]) = fa[j];
#pragma unroll
    for (int j = 0; j < 8; ++j) *reinterpret_cast<bf16x8*>(&lds_w[(frow + 32 * j) * MOE_LDS_STRIDE + 8 * piece]) = fw[j];
  };
  auto multiply = [&]() {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 a[4], w[8];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
        a[mt] = *reinterpret_cast<const bf16x8*>(&lds_a[(wr * 64 + 16 * mt + col) * MOE_LDS_STRIDE + 32 * half + 8 * kg]);
#pragma unroll
      for (int nt = 0; nt < 8; ++nt) {
        // gated: tiles 0..3 are gate's features wc * 64 + 16 nt, tiles 4..7 the same features of up
        const int row = GATED ? (nt / 4) * 128 + wc * 64 + 16 * (nt % 4) + col : wc * 128 + 16 * nt + col;
        w[nt] = *reinterpret_cast<const bf16x8*>(&lds_w[row * MOE_LDS_STRIDE + 32 * half + 8 * kg]);
      }
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[nt], a[mt], acc[mt][nt], 0, 0, 0);
    }
  };
  fetch(0);
  stage();
  __syncthreads();
  const int steps = K / MOE_BIG_K;
  for (int s = 1; s < steps; ++s) {
    fetch(MOE_BIG_K * s);  // on its way while the step before is multiplied
    multiply();
    __syncthreads();       // everyone has read the step before
    stage();
    __syncthreads();
  }
  multiply();
  // a lane holds features 16 nt + 4 kg .. + 3 (of its wavefront's) of the row wr * 64 + 16 mt + col
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int r = wr * 64 + 16 * mt + col;
    if (r >= tile.z) continue;
    if (GATED) {
      bf16_t* o = act_out + (int64_t)(tile.y + r) * N;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int f = n_base + wc * 64 + 16 * nt + 4 * kg;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (f + i < N) o[f + i] = __float2bfloat16(act_of(acc[mt][nt][i], act_kind) * acc[mt][nt + 4][i]);
      }
    } else {
      const int pair = order[tile.y + r];
      const float weight = weights[pair];
      float* o = y + ((int64_t)(pair % top) * num_tokens + pair / top) * N;
#pragma unroll
      for (int nt = 0; nt < 8; ++nt) {
        const int n = n_base + wc * 128 + 16 * nt + 4 * kg;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) o[n + i] = weight * acc[mt][nt][i];
      }
    }
  }
}

// rows a tile holds for a step of that many pairs: 16 while an expert sees a few tokens, 64 in portions, 128 in prompts
static int moe_tile_rows(int pairs, int hidden, int inter) {
  if (pairs <= 512) return 16;
  return (pairs > 4096 && hidden % MOE_BIG_K == 0 && inter % MOE_BIG_K == 0) ? MOE_BIG_ROWS : 64;
}
extern "C" int pae_moe_tile_rows(int pairs) { return pairs <= 512 ? 16 : (pairs <= 4096 ? 64 : MOE_BIG_ROWS); }
extern "C" int pae_moe_max_tiles(int pairs, int experts) {
  const int rows = pairs <= 512 ? 16 : 64;  // the smallest tiles such a step may get: the most tiles there can be
  return (pairs + rows - 1) / rows + experts;
}
extern "C" int pae_moe_tiles_supported(int hidden, int inter) { return hidden % 32 == 0 && inter % 32 == 0; }

// `order` int32 [pairs], `tiles` int32 [pae_moe_max_tiles][4], `act` bfloat16 [pairs][inter] are work space;
// y float32 [top][num_tokens][hidden] receives every pair's weighted output.
extern "C" int pae_moe_experts_tiles(float* y, const void* x, int64_t ldx, const void* gate_w, const void* up_w,
                                     const void* down_w, const int* chosen, const float* weights, int num_tokens, int top,
                                     int experts, int hidden, int inter, int act_kind, int* order, int* tiles, void* act,
                                     hipStream_t stream) {
  PAE_REQUIRE(top > 0 && experts > 0 && experts <= 4096, "experts: bad sizes top=%d experts=%d", top, experts);
  PAE_REQUIRE(pae_moe_tiles_supported(hidden, inter), "experts: widths %d and %d are no multiples of 32", hidden, inter);
  PAE_REQUIRE(ldx >= hidden && ldx % 8 == 0, "experts: row stride %lld", (long long)ldx);
  if (num_tokens <= 0) return 0;
  const int pairs = num_tokens * top;
  const int tile_rows = moe_tile_rows(pairs, hidden, inter), max_tiles = pae_moe_max_tiles(pairs, experts);
  moe_sort_kernel<<<1, 1024, (size_t)(4 * experts + 1) * sizeof(int), stream>>>(chosen, pairs, experts, tile_rows, order,
                                                                               (int4*)tiles, max_tiles);
#define MOE_TILES(MT, UP_NT, DOWN_NT)                                                                                      \
  do {                                                                                                                     \
    dim3 up_grid(max_tiles, (inter + 64 * UP_NT - 1) / (64 * UP_NT)), down_grid(max_tiles, (hidden + 64 * DOWN_NT - 1) / (64 * DOWN_NT)); \
    PAE_REQUIRE(up_grid.y <= 65535 && down_grid.y <= 65535, "experts: widths %d, %d exceed the grid", hidden, inter);      \
    moe_tiles_gate_up_kernel<MT, UP_NT><<<up_grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)x, ldx,                   \
                                                                      (const bf16_t*)gate_w, (const bf16_t*)up_w, order,    \
                                                                      (const int4*)tiles, top, hidden, inter, act_kind);    \
    moe_tiles_down_kernel<MT, DOWN_NT><<<down_grid, 256, 0, stream>>>(y, (const bf16_t*)act, (const bf16_t*)down_w, order,  \
                                                                       weights, (const int4*)tiles, top, num_tokens, hidden, \
                                                                       inter);                                              \
  } while (0)
  if (tile_rows == 16) {
    dim3 up_grid(max_tiles, (inter + 15) / 16), down_grid(max_tiles, (hidden + 15) / 16);
    PAE_REQUIRE(up_grid.y <= 65535 && down_grid.y <= 65535, "experts: widths %d, %d exceed the grid", hidden, inter);
    moe_few_tiles_kernel<true><<<up_grid, 256, 0, stream>>>((bf16_t*)act, nullptr, (const bf16_t*)x, ldx, (const bf16_t*)gate_w,
                                                            (const bf16_t*)up_w, order, weights, (const int4*)tiles, top,
                                                            num_tokens, hidden, inter, act_kind);
    moe_few_tiles_kernel<false><<<down_grid, 256, 0, stream>>>(nullptr, y, (const bf16_t*)act, inter, (const bf16_t*)down_w,
                                                               nullptr, order, weights, (const int4*)tiles, top, num_tokens,
                                                               inter, hidden, act_kind);
  } else if (tile_rows == 64) MOE_TILES(4, 2, 4);
  else {
    dim3 up_grid(max_tiles, (inter + 127) / 128), down_grid(max_tiles, (hidden + 255) / 256);
    PAE_REQUIRE(up_grid.y <= 65535 && down_grid.y <= 65535, "experts: widths %d, %d exceed the grid", hidden, inter);
    moe_big_tiles_kernel<true><<<up_grid, 256, 0, stream>>>((bf16_t*)act, nullptr, (const bf16_t*)x, ldx, (const bf16_t*)gate_w,
                                                            (const bf16_t*)up_w, order, weights, (const int4*)tiles, top,
                                                            num_tokens, hidden, inter, act_kind);
    moe_big_tiles_kernel<false><<<down_grid, 256, 0, stream>>>(nullptr, y, (const bf16_t*)act, inter, (const bf16_t*)down_w,
                                                               nullptr, order, weights, (const int4*)tiles, top, num_tokens,
                                                               inter, hidden, act_kind);
  }
#undef MOE_TILES
  return pae_check_launch("moe_experts_tiles");
}
