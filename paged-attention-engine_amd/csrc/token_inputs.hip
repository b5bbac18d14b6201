// What a token brings besides its embedding row: a learned row for its position, and, layer by layer, a few
// columns of a second token table that gate a narrow product of the stream.
//
//   embedding_positions   out[t] = scale * table[ids[t]] + rows[positions[t]]  (float32; the position's row unscaled)
//   token_gate            out[t][i] = T(act(gate[t][i]) * columns[ids[t]][i]): `gate` is a narrow product of the
//                         stream, `columns` [vocab][dim] the layer's share of the second table; the activation
//                         (0 gelu by erf, 1 gelu by tanh, 2 silu) and the product are float32, rounded once
//   token_side_rows       for steps of a few rows, the whole of a layer's token input in one launch, a workgroup a row:
//                         g = T(act(T(W_gate x)) * columns[id]);  y = W_proj g;  stream += y / sqrt(mean(y^2) + eps) * w,
//                         and, as asked, the new stream normed for the next reader.  x is the stream in the activation
//                         type; sums are float32, and g is rounded where the separate products would round it
#include "common.h"
#include "api.h"

template <typename T>
__global__ void embedding_positions_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids,
                                           const T* __restrict__ rows, const int* __restrict__ positions, int hidden,
                                           float scale) {
  const int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * hidden;
  const T* place = rows + (int64_t)positions[t] * hidden;
  float* dst = out + (int64_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = scale * to_f32(row[i]) + to_f32(place[i]);
}

extern "C" int pae_embedding_positions(int dtype, float* out, const void* table, const int* ids, const void* rows,
                                       const int* positions, int num_tokens, int hidden, int vocab, float scale,
                                       hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0, "embedding with positions: bad sizes T=%d H=%d V=%d", num_tokens,
              hidden, vocab);
  PAE_REQUIRE(table && rows && ids && positions, "embedding with positions: a table, the rows of positions and both index lists are needed");
  if (num_tokens == 0) return 0;
  if (dtype == PAE_F32)
    embedding_positions_kernel<float><<<num_tokens, 256, 0, stream>>>(out, (const float*)table, ids, (const float*)rows,
                                                                      positions, hidden, scale);
  else if (dtype == PAE_BF16)
    embedding_positions_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(out, (const bf16_t*)table, ids, (const bf16_t*)rows,
                                                                       positions, hidden, scale);
  else
    return pae_fail("embedding with positions: unknown dtype code %d", dtype);
  return pae_check_launch("embedding_positions");
}

template <typename T>
__global__ __launch_bounds__(256) void token_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, int64_t gate_stride,
                                                         const T* __restrict__ columns, const int* __restrict__ ids,
                                                         int dim, int kind, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / dim;
  const int i = (int)(idx % dim);
  out[idx] = from_f32<T>(act_of(to_f32(gate[t * gate_stride + i]), kind) * to_f32(columns[(int64_t)ids[t] * dim + i]));
}

extern "C" int pae_token_gate(int dtype, void* out, const void* gate, int64_t gate_stride, const void* columns,
                              const int* ids, int num_tokens, int dim, int kind, hipStream_t stream) {
  PAE_REQUIRE(dim > 0 && gate_stride >= dim, "token gate: %d columns in rows of %lld", dim, (long long)gate_stride);
  PAE_REQUIRE(kind >= 0 && kind <= 2, "token gate: unknown activation code %d", kind);
  if (num_tokens <= 0) return 0;
  const int64_t total = (int64_t)num_tokens * dim;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == PAE_F32)
    token_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gate, gate_stride, (const float*)columns,
                                                         ids, dim, kind, total);
  else if (dtype == PAE_BF16)
    token_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate, gate_stride,
                                                          (const bf16_t*)columns, ids, dim, kind, total);
  else
    return pae_fail("token gate: unknown dtype code %d", dtype);
  return pae_check_launch("token_gate");
}

// One workgroup of four wavefronts per row.  The gate's `dim` outputs are dealt to the wavefronts in turn (a wavefront's
// lanes share out the width and meet in a fixed order); then a thread takes output features of the second product in
// turn, each a sum over the `dim` gated columns in ascending order; the row's sums of squares meet through LDS.
template <typename T>
__global__ __launch_bounds__(256) void token_side_rows_kernel(
    float* __restrict__ residual, const T* __restrict__ rows, int64_t row_stride, const T* __restrict__ gate_w,
    const T* __restrict__ columns, const int* __restrict__ ids, const T* __restrict__ proj_w, int kind,
    const void* __restrict__ w_out, int w_out_is_f32, float eps, const void* __restrict__ w_next, int w_next_is_f32,
    float eps_next, T* __restrict__ normed, int hidden, int dim) {
  extern __shared__ float side_lds[];  // [hidden] the row, then the new stream; [dim] the gated columns
  __shared__ float scratch[4];
  float* x_lds = side_lds;
  float* g_lds = side_lds + hidden;
  const int64_t t = blockIdx.x;
  const T* x = rows + t * row_stride;
  for (int i = threadIdx.x; i < hidden; i += 256) x_lds[i] = to_f32(x[i]);
  __syncthreads();
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  const T* mine = columns + (int64_t)ids[t] * dim;
  for (int j = wave; j < dim; j += 4) {
    const T* w = gate_w + (int64_t)j * hidden;
    float sum = 0.f;
    for (int k = lane; k < hidden; k += PAE_WAVE) sum = fmaf(x_lds[k], to_f32(w[k]), sum);
    sum = wave_sum(sum);
    if (lane == 0) g_lds[j] = round_to<T>(act_of(round_to<T>(sum), kind) * to_f32(mine[j]));
  }
  __syncthreads();
  float* res = residual + t * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const T* w = proj_w + (int64_t)i * dim;
    float sum = 0.f;
    for (int k = 0; k < dim; ++k) sum = fmaf(g_lds[k], to_f32(w[k]), sum);
    x_lds[i] = sum;  // the row of x has been used up: its place takes y
    ss = fmaf(sum, sum, ss);
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  float sx = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float v = res[i] + x_lds[i] * inv * load_param(w_out, w_out_is_f32, i);
    res[i] = v;
    x_lds[i] = v;
    sx = fmaf(v, v, sx);
  }
  if (!normed) return;
  sx = block_sum<4>(sx, scratch);
  const float inv_next = 1.0f / sqrtf(sx / (float)hidden + eps_next);
  for (int i = threadIdx.x; i < hidden; i += 256)
    normed[t * hidden + i] = from_f32<T>(x_lds[i] * inv_next * load_param(w_next, w_next_is_f32, i));
}

extern "C" int pae_token_side_rows(int dtype, float* residual, const void* rows, int64_t row_stride, const void* gate_w,
                                   const void* columns, const int* ids, const void* proj_w, int kind, const void* w_out,
                                   int w_out_is_f32, float eps, const void* w_next, int w_next_is_f32, float eps_next,
                                   void* normed, int num_rows, int hidden, int dim, hipStream_t stream) {
  PAE_REQUIRE(hidden > 0 && dim > 0 && row_stride >= hidden, "token side: bad sizes H=%d dim=%d", hidden, dim);
  PAE_REQUIRE((size_t)(hidden + dim) * sizeof(float) <= 60 * 1024, "token side: a row of %d and %d columns exceed the kernel's LDS",
              hidden, dim);
  PAE_REQUIRE(kind >= 0 && kind <= 2, "token side: unknown activation code %d", kind);
  PAE_REQUIRE(w_out && (!normed || w_next), "token side: a norm without its weight");
  if (num_rows <= 0) return 0;
  const size_t lds = (size_t)(hidden + dim) * sizeof(float);
  if (dtype == PAE_F32)
    token_side_rows_kernel<float><<<num_rows, 256, lds, stream>>>(
        residual, (const float*)rows, row_stride, (const float*)gate_w, (const float*)columns, ids, (const float*)proj_w, kind,
        w_out, w_out_is_f32, eps, w_next, w_next_is_f32, eps_next, (float*)normed, hidden, dim);
  else if (dtype == PAE_BF16)
    token_side_rows_kernel<bf16_t><<<num_rows, 256, lds, stream>>>(
        residual, (const bf16_t*)rows, row_stride, (const bf16_t*)gate_w, (const bf16_t*)columns, ids, (const bf16_t*)proj_w,
        kind, w_out, w_out_is_f32, eps, w_next, w_next_is_f32, eps_next, (bf16_t*)normed, hidden, dim);
  else
    return pae_fail("token side: unknown dtype code %d", dtype);
  return pae_check_launch("token_side_rows");
}
