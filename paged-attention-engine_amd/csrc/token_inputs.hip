// What a token brings besides its embedding row: a learned row for its position, and, layer by layer, a few
// columns of a second token table that gate a narrow product of the stream.
//
//   embedding_positions   out[t] = scale * table[ids[t]] + rows[positions[t]]  (float32; the position's row unscaled)
//   token_gate            out[t][i] = T(act(gate[t][i]) * columns[ids[t]][i]): `gate` is a narrow product of the
//                         stream, `columns` [vocab][dim] the layer's share of the second table; the activation
//                         (0 gelu by erf, 1 gelu by tanh, 2 silu) and the product are float32, rounded once
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
