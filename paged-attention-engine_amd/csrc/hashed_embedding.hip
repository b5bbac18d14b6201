// The embedding with a hashed table of token pairs added to it.
//
// out[t] = scale * table[id_t] + pairs[row_t], float32, where row_t = (prev_t * mul_prev + id_t * mul_cur) mod
// buckets and prev_t is the token before id_t in its own sequence; a sequence's first token (position
// 0) takes the table's last row, number `buckets`.  The token before a step's first row of a
// sequence is per-request state, last_token[slot]; it is read here and moved on by a second kernel
// once every row has read it (a sequence's rows are consecutive in the step, in order).
#include "common.h"
#include "api.h"

template <typename T>
__global__ void embedding_pairs_kernel(float* __restrict__ out, const T* __restrict__ table, const T* __restrict__ pairs,
                                       const int* __restrict__ ids, const int* __restrict__ positions,
                                       const int* __restrict__ tok_seq, const int* __restrict__ slots,
                                       const int* __restrict__ last_token, int hidden, float scale, int buckets,
                                       int mul_prev, int mul_cur) {
  const int t = blockIdx.x;
  const int id = ids[t], s = tok_seq[t];
  int64_t row = buckets;
  if (positions[t] > 0) {
    const int prev = (t > 0 && tok_seq[t - 1] == s) ? ids[t - 1] : last_token[slots[s]];
    row = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const T* a = table + (int64_t)id * hidden;
  const T* b = pairs + row * hidden;
  float* o = out + (int64_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = scale * to_f32(a[i]) + to_f32(b[i]);
}

__global__ void last_token_kernel(const int* __restrict__ ids, const int* __restrict__ tok_seq, const int* __restrict__ slots,
                                  int* __restrict__ last_token, int num_tokens) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= num_tokens) return;
  const int s = tok_seq[t];
  if (t == num_tokens - 1 || tok_seq[t + 1] != s) last_token[slots[s]] = ids[t];
}

extern "C" int pae_embedding_pairs(int dtype, float* out, const void* table, const void* pair_table, const int* ids,
                                   const int* positions, const int* tok_seq, const int* slots, int* last_token,
                                   int num_tokens, int hidden, int vocab, float scale, int buckets, int mul_prev,
                                   int mul_cur, hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0 && buckets > 0, "pair embedding: bad sizes T=%d H=%d V=%d buckets=%d",
              num_tokens, hidden, vocab, buckets);
  PAE_REQUIRE(mul_prev >= 0 && mul_cur >= 0, "pair embedding: negative multipliers %d, %d", mul_prev, mul_cur);
  if (num_tokens == 0) return 0;
  if (dtype == PAE_F32)
    embedding_pairs_kernel<float><<<num_tokens, 256, 0, stream>>>(out, (const float*)table, (const float*)pair_table, ids,
                                                                  positions, tok_seq, slots, last_token, hidden, scale,
                                                                  buckets, mul_prev, mul_cur);
  else if (dtype == PAE_BF16)
    embedding_pairs_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(out, (const bf16_t*)table, (const bf16_t*)pair_table,
                                                                   ids, positions, tok_seq, slots, last_token, hidden,
                                                                   scale, buckets, mul_prev, mul_cur);
  else
    return pae_fail("pair embedding: unknown dtype code %d", dtype);
  last_token_kernel<<<(num_tokens + 255) / 256, 256, 0, stream>>>(ids, tok_seq, slots, last_token, num_tokens);
  return pae_check_launch("embedding_pairs");
}
