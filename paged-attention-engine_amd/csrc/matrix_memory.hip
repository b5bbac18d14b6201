// A matrix memory with exponential gates: a recurrent mixer whose per-request state is, per head, a matrix
// C [D, V], the sum of its gated keys n [D] and a running maximum m of the gates' logarithms.
//
// A step's projected rows hold, per token, [q: H heads of D | k: H heads of D | v: H heads of V]; `gate_logits`
// [T][2H] are the float32 sums of the two gate projections with their biases.  With cap c:
//
//   i = c tanh(z_i / c);   f = logsigmoid(c tanh(z_f / c));   m_t = max(f + m_(t-1), i)
//   keep = exp(f + m_(t-1) - m_t);   take = exp(i - m_t)
//   C <- keep C + take k v^T;   n <- keep n + take k
//   o = C^T q / (max(|n . q|, exp(-m_t)) + floor_eps),  q times D^-1/2
//
// then o is divided by its root mean square over V, multiplied by a weight (one per head and feature) and by
// sigmoid(gate), and rounded to the activation type.  m starts at 0 like C and n (a slot is zeroed when
// a request takes it).  n is kept as one more column of C, whose "value" is 1 for every token, so the
// recurrence is the delta rule's kernel without its read-before-write (delta_rule.hip), over V + 1
// columns.  Three kernels around it:
//
//   memory_prepare   q, k, v to float32 rows (q scaled, v with its column of ones)
//   memory_gates     one wavefront per (sequence, head): 64 tokens' gate logarithms at a time, the chain
//                    of maxima walked by all lanes together, then each lane its token's keep and take
//   memory_finish    the division, the norm over V, weight and gate
//
// Everything but the projected rows and the gate's rows is float32.
#include "common.h"
#include "api.h"

void pae_launch_recurrence(const float* q, const float* k, const float* v, const float* beta, const float* decay,
                           const int4* runs, const int* slots, float* state, int64_t state_slot_stride, int G, int H,
                           int D, int V, int num_seqs, int channel_decay, int delta, float* o, hipStream_t stream);

template <typename T>
__global__ __launch_bounds__(128) void memory_prepare_kernel(const T* __restrict__ proj, int64_t row_stride, int H, int D,
                                                             int V, float* __restrict__ q_out, float* __restrict__ k_out,
                                                             float* __restrict__ v_out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const T* row = proj + t * row_stride;
  const float q_scale = 1.0f / sqrtf((float)D);
  for (int d = threadIdx.x; d < D; d += 128) {
    q_out[(t * H + h) * D + d] = to_f32(row[h * D + d]) * q_scale;
    k_out[(t * H + h) * D + d] = to_f32(row[(H + h) * D + d]);
  }
  float* v = v_out + (t * H + h) * (V + 1);
  for (int i = threadIdx.x; i < V; i += 128) v[i] = to_f32(row[2 * H * D + h * V + i]);
  if (threadIdx.x == 0) v[V] = 1.0f;
}

__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

__global__ __launch_bounds__(PAE_WAVE) void memory_gates_kernel(const float* __restrict__ gate_logits, const int4* __restrict__ seq_runs,
                                                                const int* __restrict__ slots, float* __restrict__ maximum,
                                                                int64_t max_slot_stride, int H, float cap,
                                                                float* __restrict__ take_out, float* __restrict__ keep_out,
                                                                float* __restrict__ floor_out) {
  const int s = blockIdx.y, h = blockIdx.x, lane = threadIdx.x;
  const int4 run = seq_runs[s];
  float* m_at = maximum + (int64_t)slots[s] * max_slot_stride + h;
  float m = *m_at;
  for (int first = 0; first < run.y; first += PAE_WAVE) {
    const int n = min(PAE_WAVE, run.y - first);
    const int64_t t = run.x + first + lane;
    float li = 0.f, lf = 0.f;
    if (lane < n) {
      li = cap * tanhf(gate_logits[t * 2 * H + h] / cap);
      lf = log_sigmoid_f(cap * tanhf(gate_logits[t * 2 * H + H + h] / cap));
    }
    float before = 0.f, after = 0.f;  // the maximum before and after this lane's token
    for (int j = 0; j < n; ++j) {
      const float fj = __shfl(lf, j, PAE_WAVE), ij = __shfl(li, j, PAE_WAVE);
      const float next = fmaxf(fj + m, ij);
      if (lane == j) {
        before = m;
        after = next;
      }
      m = next;
    }
    if (lane < n) {
      keep_out[t * H + h] = expf(lf + before - after);
      take_out[t * H + h] = expf(li - after);
      floor_out[t * H + h] = expf(-after);
    }
  }
  if (lane == 0) *m_at = m;
}

template <typename T>
__global__ __launch_bounds__(PAE_WAVE) void memory_finish_kernel(const float* __restrict__ o, const float* __restrict__ floors,
                                                                 const T* __restrict__ gates, int64_t gate_stride,
                                                                 const void* __restrict__ weight, int w_is_f32, float eps,
                                                                 float floor_eps, int H, int V, T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + (t * H + h) * (V + 1);
  const float denom = fmaxf(fabsf(x[V]), floors[t * H + h]) + floor_eps;
  float ss = 0.f;
  for (int i = lane; i < V; i += PAE_WAVE) {
    const float y = x[i] / denom;
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + eps);
  const T* gate = gates + t * gate_stride + h * V;
  for (int i = lane; i < V; i += PAE_WAVE) {
    const float g = 1.0f / (1.0f + expf(-to_f32(gate[i])));
    out[(t * H + h) * V + i] = from_f32<T>(x[i] / denom * inv * load_param(weight, w_is_f32, h * V + i) * g);
  }
}

extern "C" int pae_matrix_memory_step(int dtype, const void* proj, int64_t row_stride, const void* gate_in,
                                      int64_t gate_stride, const float* gate_logits, int num_tokens, int num_seqs,
                                      const int* seq_runs, const int* slots, int H, int D, int V, float gate_cap,
                                      float* state, int64_t state_slot_stride, float* maximum, int64_t max_slot_stride,
                                      const void* norm_w, int w_is_f32, float norm_eps, float floor_eps, float* work,
                                      void* out, hipStream_t stream) {
  PAE_REQUIRE(H > 0 && D > 0 && V > 0, "matrix memory: bad head sizes H=%d D=%d V=%d", H, D, V);
  PAE_REQUIRE(D <= 1024 && V <= 1023, "matrix memory: key width %d or value width %d exceeds the kernels' limits", D, V);
  PAE_REQUIRE(H <= 65535 && num_seqs <= 65535, "matrix memory: %d heads, %d sequences exceed the grid", H, num_seqs);
  PAE_REQUIRE(row_stride >= 2 * (int64_t)H * D + (int64_t)H * V, "matrix memory: row stride %lld too small", (long long)row_stride);
  PAE_REQUIRE(gate_cap > 0.f, "matrix memory: the gates' cap must be positive, got %g", (double)gate_cap);
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "matrix memory: unknown dtype code %d", dtype);
  if (num_tokens <= 0 || num_seqs <= 0) return 0;
  // work: q [T][H][D], k [T][H][D], v [T][H][V + 1], take [T][H], keep [T][H], floor [T][H], o [T][H][V + 1]
  float* q = work;
  float* k = q + (int64_t)num_tokens * H * D;
  float* v = k + (int64_t)num_tokens * H * D;
  float* take = v + (int64_t)num_tokens * H * (V + 1);
  float* keep = take + (int64_t)num_tokens * H;
  float* floors = keep + (int64_t)num_tokens * H;
  float* o = floors + (int64_t)num_tokens * H;
  const int4* runs = (const int4*)seq_runs;
  dim3 token_heads(num_tokens, H);
  memory_gates_kernel<<<dim3(H, num_seqs), PAE_WAVE, 0, stream>>>(gate_logits, runs, slots, maximum, max_slot_stride, H,
                                                                   gate_cap, take, keep, floors);
#define MEMORY_LAUNCH(T)                                                                                              \
  memory_prepare_kernel<T><<<token_heads, 128, 0, stream>>>((const T*)proj, row_stride, H, D, V, q, k, v);            \
  pae_launch_recurrence(q, k, v, take, keep, runs, slots, state, state_slot_stride, H, H, D, V + 1, num_seqs, 0, 0, o, \
                        stream);                                                                                      \
  memory_finish_kernel<T><<<token_heads, PAE_WAVE, 0, stream>>>(o, floors, (const T*)gate_in, gate_stride, norm_w,    \
                                                                w_is_f32, norm_eps, floor_eps, H, V, (T*)out)
  if (dtype == PAE_F32) {
    MEMORY_LAUNCH(float);
  } else {
    MEMORY_LAUNCH(bf16_t);
  }
#undef MEMORY_LAUNCH
  return pae_check_launch("matrix_memory_step");
}

// floats of `work` that pae_matrix_memory_step needs for a step of `num_tokens` rows
extern "C" int64_t pae_matrix_memory_work_floats(int num_tokens, int H, int D, int V) {
  return (int64_t)num_tokens * H * (2 * (int64_t)D + 2 * ((int64_t)V + 1) + 3);
}
