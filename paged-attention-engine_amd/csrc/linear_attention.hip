// Gated linear attention: a recurrent mixer whose per-request state is one matrix S [D, V] per head, which
// decays per token by a factor of its own for every key channel (every row of S):
//
//   a_t = sigmoid(z_t + bias)^(1 / tau)          (one number per head and key channel)
//   S  <- diag(a_t) S + k_t v_t^T;   o_t = S^T q_t,   q times D^-1/2
//
// then o is divided by its root mean square over V, multiplied by a weight of V numbers that the heads share
// and by act(gate) (SiLU or sigmoid), and rounded to the activation type.  S starts at zero (a slot is zeroed
// when a request takes it).  A step's projected rows hold, per token, [q: H heads of D | k: H heads of D |
// v: H heads of V]; the decay's input z [T][H D] and the gate's rows [T][H V] come as rows of their own.  Three
// kernels:
//
//   gla_prepare      q, k, v to float32 rows (q scaled); the decays as exp(logsigmoid(z + bias) / tau)
//   the delta rule's recurrence kernel (delta_rule.hip) with a decay per key channel and without its
//   read-before-write: a column of S stays in the registers of a group of lanes over the whole step
//   the delta rule's gated norm
//
// Everything but the projected rows, z and the gate's rows is float32: the decay and its logarithm, the state,
// the read-out and the norm.  The order in which a column's sums are formed depends on D alone, so a token's
// result does not depend on how a prompt was cut into steps or on what else the step holds.
#include "common.h"
#include "api.h"

void pae_launch_recurrence(const float* q, const float* k, const float* v, const float* beta, const float* decay,
                           const int4* runs, const int* slots, float* state, int64_t state_slot_stride, int G, int H,
                           int D, int V, int num_seqs, int channel_decay, int delta, float* o, hipStream_t stream);
int pae_launch_gated_norm(int dtype, const float* o, const void* gates, int64_t gate_stride, int gate_sigmoid,
                          const void* weight, int w_is_f32, float eps, int num_tokens, int H, int V, void* out,
                          hipStream_t stream);

__device__ __forceinline__ float gla_log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One workgroup of 128 threads per (token, head).
template <typename T>
__global__ __launch_bounds__(128) void gla_prepare_kernel(const T* __restrict__ proj, int64_t row_stride,
                                                          const T* __restrict__ z_in, int64_t z_stride,
                                                          const void* __restrict__ z_bias, int bias_is_f32, float inv_tau,
                                                          int H, int D, int V, float* __restrict__ q_out,
                                                          float* __restrict__ k_out, float* __restrict__ v_out,
                                                          float* __restrict__ decay_out, float* __restrict__ ones_out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const T* row = proj + t * row_stride;
  const T* z = z_in + t * z_stride + h * D;
  const float q_scale = 1.0f / sqrtf((float)D);
  const int64_t at = (t * H + h) * D;
  for (int d = threadIdx.x; d < D; d += 128) {
    q_out[at + d] = to_f32(row[h * D + d]) * q_scale;
    k_out[at + d] = to_f32(row[(H + h) * D + d]);
    const float bias = z_bias ? load_param(z_bias, bias_is_f32, h * D + d) : 0.f;
    decay_out[at + d] = expf(gla_log_sigmoid(to_f32(z[d]) + bias) * inv_tau);
  }
  float* v = v_out + (t * H + h) * V;
  for (int i = threadIdx.x; i < V; i += 128) v[i] = to_f32(row[2 * H * D + h * V + i]);
  if (threadIdx.x == 0) ones_out[t * H + h] = 1.0f;  // the recurrence's write strength: every token writes k v^T whole
}

static int64_t gla_part(int64_t floats) { return (floats + 3) / 4 * 4; }

extern "C" int pae_linear_attention_step(int dtype, const void* proj, int64_t row_stride, const void* z_in, int64_t z_stride,
                                         const void* z_bias, int bias_is_f32, float tau, const void* gate_in,
                                         int64_t gate_stride, int gate_sigmoid, int num_tokens, int num_seqs,
                                         const int* seq_runs, const int* slots, int H, int D, int V, float* state,
                                         int64_t state_slot_stride, const void* norm_w, int w_is_f32, float norm_eps,
                                         float* work, void* out, hipStream_t stream) {
  PAE_REQUIRE(H > 0 && D > 0 && V > 0, "linear attention: bad head sizes H=%d D=%d V=%d", H, D, V);
  PAE_REQUIRE(D <= 1024 && V <= 1024, "linear attention: key width %d or value width %d exceeds 1024", D, V);
  PAE_REQUIRE(H <= 65535 && num_seqs <= 65535, "linear attention: %d heads, %d sequences exceed the grid", H, num_seqs);
  PAE_REQUIRE(row_stride >= 2 * (int64_t)H * D + (int64_t)H * V, "linear attention: row stride %lld too small", (long long)row_stride);
  PAE_REQUIRE(z_stride >= (int64_t)H * D && gate_stride >= (int64_t)H * V, "linear attention: the decay's or the gate's rows are too narrow");
  PAE_REQUIRE(tau > 0.f, "linear attention: the decay's temperature must be positive, got %g", (double)tau);
  PAE_REQUIRE(z_in && gate_in, "linear attention: the decay's and the gate's rows are needed");
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "linear attention: unknown dtype code %d", dtype);
  if (num_tokens <= 0 || num_seqs <= 0) return 0;
  // work: q [T][H][D], k [T][H][D], decay [T][H][D], v [T][H][V], ones [T][H], o [T][H][V], each on a 16-byte boundary
  const int64_t T = num_tokens;
  float* q = work;
  float* k = q + gla_part(T * H * D);
  float* decay = k + gla_part(T * H * D);
  float* v = decay + gla_part(T * H * D);
  float* ones = v + gla_part(T * H * V);
  float* o = ones + gla_part(T * H);
  const int4* runs = (const int4*)seq_runs;
  dim3 token_heads(num_tokens, H);
  if (dtype == PAE_F32)
    gla_prepare_kernel<float><<<token_heads, 128, 0, stream>>>((const float*)proj, row_stride, (const float*)z_in, z_stride,
                                                               z_bias, bias_is_f32, 1.0f / tau, H, D, V, q, k, v, decay, ones);
  else
    gla_prepare_kernel<bf16_t><<<token_heads, 128, 0, stream>>>((const bf16_t*)proj, row_stride, (const bf16_t*)z_in, z_stride,
                                                                z_bias, bias_is_f32, 1.0f / tau, H, D, V, q, k, v, decay, ones);
  pae_launch_recurrence(q, k, v, ones, decay, runs, slots, state, state_slot_stride, H, H, D, V, num_seqs, 1, 0, o, stream);
  const int code = pae_launch_gated_norm(dtype, o, gate_in, gate_stride, gate_sigmoid, norm_w, w_is_f32, norm_eps,
                                         num_tokens, H, V, out, stream);
  if (code) return code;
  return pae_check_launch("linear_attention_step");
}

// floats of `work` that pae_linear_attention_step needs for a step of `num_tokens` rows
extern "C" int64_t pae_linear_attention_work_floats(int num_tokens, int H, int D, int V) {
  const int64_t T = num_tokens;
  return 3 * gla_part(T * H * D) + 2 * gla_part(T * H * V) + gla_part(T * H);
}
