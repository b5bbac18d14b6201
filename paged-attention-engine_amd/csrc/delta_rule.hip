// The gated delta rule: a recurrent mixer whose per-request state is one matrix per head and the
// last few inputs of its short convolutions.
//
// A step's projected rows hold, per token,
//   [q: G heads of D | k: G heads of D | v: H heads of V | gate: H heads of V | b: H | a: H]
// (G key heads serve H value heads, head h reads key head h / (H / G)).  Four kernels:
//
//   delta_prepare      the first C = 2 G D + H V columns pass a causal convolution over time, one
//                      filter of `taps` taps per column (the last tap is the current token's; what
//                      came before the step is read from the request's state, zeros at its start),
//                      and SiLU; q and k heads become unit vectors, x / sqrt(sum x^2 + unit_eps), q
//                      also times D^-1/2; beta = sigmoid(b); decay = exp(-exp(A_log) softplus(a + dt)).
//   delta_conv_tail    the state's last taps - 1 inputs are moved on by the step's rows.
//   delta_recurrence   per head and token, in this order:  S <- decay S;  u = beta (v - S^T k);
//                      S <- S + k u^T;  o = S^T q.  Columns of S are independent of each other, so a
//                      column is owned by a group of lanes that hold it in registers from the step's
//                      first token to its last; the lanes of a group share out the D rows.
//   delta_gated_norm   o / sqrt(mean_V(o^2) + eps) * w * silu(gate), rounded to the activation type.
//
// For designs that have them, each switched by a parameter: a decay per head and key channel instead of one
// per head (`channel_decay`: the decay's input and dt_bias are then H x D wide and row d of a head's S is
// multiplied by its own number); beta, the decay's input and the gate read from rows of their own instead of
// the projected rows' tail (a design whose decay and gate pass through a narrow product first); sigmoid
// instead of SiLU on the gate.  The recurrence kernels also run a matrix memory that only adds
// (`delta` off: u = beta v, nothing is read back before the write; see matrix_memory.hip).
//
// Everything but the projected rows is float32: the convolution's sums, the unit vectors, beta,
// the decay and its logarithm, the state, the read-out and the norm.  The order in which a
// column's sums are formed depends on D alone, so a token's result does not depend on how a
// prompt was cut into steps or on what else the step holds.
#include "common.h"
#include "api.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// seq_runs[s] = (first flat row, rows in this step, tokens held before the step, unused)
// One workgroup of 128 threads per (token, segment): segments 0 .. G-1 are the q heads, G .. 2G-1 the
// k heads, 2G .. 2G+H-1 the v heads; the workgroup of segment 0 also computes the token's beta and decay.
template <typename T>
__global__ __launch_bounds__(128) void delta_prepare_kernel(
    const T* __restrict__ proj, int64_t row_stride, const int* __restrict__ tok_seq, const int* __restrict__ positions,
    const int4* __restrict__ seq_runs, const int* __restrict__ slots, const float* __restrict__ conv_w,
    const float* __restrict__ conv_tail, int64_t tail_slot_stride, int taps, int G, int H, int D, int V,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float unit_eps, const T* __restrict__ b_in,
    int64_t b_stride, const T* __restrict__ a_in, int64_t a_stride, int channel_decay, float* __restrict__ q_out,
    float* __restrict__ k_out, float* __restrict__ v_out, float* __restrict__ beta_out, float* __restrict__ decay_out) {
  __shared__ float scratch[2];
  const int t = blockIdx.x, seg = blockIdx.y;
  const int s = tok_seq[t];
  const int4 run = seq_runs[s];
  const int in_step = t - run.x;  // rows of this sequence before this one in the step
  const int C = 2 * G * D + H * V;
  const float* tail = conv_tail + (int64_t)slots[s] * tail_slot_stride;  // [taps - 1][C], oldest first
  const bool is_v = seg >= 2 * G;
  const int width = is_v ? V : D;
  const int c0 = is_v ? 2 * G * D + (seg - 2 * G) * V : seg * D;  // the segment's first channel
  float* dst = is_v ? v_out + ((int64_t)t * H + seg - 2 * G) * V
                    : (seg < G ? q_out + ((int64_t)t * G + seg) * D : k_out + ((int64_t)t * G + seg - G) * D);
  // channels i, i + 128, ... of the segment: convolved and activated; up to 8 a thread are kept (widths to 1,024)
  float mine[8];
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const int i = threadIdx.x + 128 * n;
    mine[n] = 0.f;
    if (i >= width) break;
    const int c = c0 + i;
    float sum = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;  // tap j weighs the input `back` tokens ago
      float x;
      if (back <= in_step) x = to_f32(proj[(int64_t)(t - back) * row_stride + c]);
      else x = tail[(int64_t)(taps - 1 - (back - in_step)) * C + c];
      sum = fmaf(conv_w[(int64_t)c * taps + j], x, sum);
    }
    mine[n] = silu_f(sum);
    ss = fmaf(mine[n], mine[n], ss);
  }
  float inv = 1.f;
  const float q_scale = 1.0f / sqrtf((float)D);
  if (!is_v) {  // q and k heads become unit vectors; q is also divided by sqrt(D)
    ss = block_sum<2>(ss, scratch);
    inv = 1.0f / sqrtf(ss + unit_eps);
  }
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const int i = threadIdx.x + 128 * n;
    if (i >= width) break;
    dst[i] = is_v ? mine[n] : (seg < G ? mine[n] * inv * q_scale : mine[n] * inv);
  }
  if (seg == 0) {
    const T* b_row = b_in + (int64_t)t * b_stride;
    const T* a_row = a_in + (int64_t)t * a_stride;
    for (int h = threadIdx.x; h < H; h += 128) beta_out[(int64_t)t * H + h] = 1.0f / (1.0f + expf(-to_f32(b_row[h])));
    if (!channel_decay) {
      for (int h = threadIdx.x; h < H; h += 128)
        decay_out[(int64_t)t * H + h] = expf(-expf(a_log[h]) * softplus_f(to_f32(a_row[h]) + dt_bias[h]));
    }
  }
  if (channel_decay) {  // one decay per head and key channel, [H][D]: every segment's workgroup takes its share
    const T* a_row = a_in + (int64_t)t * a_stride;
    for (int c = seg * 128 + threadIdx.x; c < H * D; c += gridDim.y * 128)
      decay_out[(int64_t)t * H * D + c] = expf(-expf(a_log[c / D]) * softplus_f(to_f32(a_row[c]) + dt_bias[c]));
  }
}

template <typename T>
__global__ void delta_conv_tail_kernel(const T* __restrict__ proj, int64_t row_stride, const int4* __restrict__ seq_runs,
                                       const int* __restrict__ slots, float* __restrict__ conv_tail,
                                       int64_t tail_slot_stride, int taps, int C) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int4 run = seq_runs[s];
  float* tail = conv_tail + (int64_t)slots[s] * tail_slot_stride;
  const int keep = taps - 1, n = run.y;
  // entry j of the new tail is the input at (end of step) - keep + j: a row of this step, or an entry
  // further on in the old tail (read before any entry at or above it is written: j ascends)
  for (int j = 0; j < keep; ++j) {
    const int r = n - keep + j;  // row of the step, negative: before it
    tail[(int64_t)j * C + c] = r >= 0 ? to_f32(proj[(int64_t)(run.x + r) * row_stride + c]) : tail[(int64_t)(j + n) * C + c];
  }
}

// One group of L lanes per column of S; a lane holds R consecutive rows of its column.
template <int R>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ beta,
    const float* __restrict__ decay, const int4* __restrict__ seq_runs, const int* __restrict__ slots,
    float* __restrict__ state, int64_t state_slot_stride, int G, int H, int D, int V, int L, int channel_decay, int delta,
    float* __restrict__ out) {
  const int s = blockIdx.z, h = blockIdx.y;
  const int col = blockIdx.x * (256 / L) + threadIdx.x / L;
  const int sub = threadIdx.x % L;
  const int4 run = seq_runs[s];
  if (col >= V) return;  // whole groups leave together: the shuffles below stay within a group
  const int g = h / (H / G);
  float* column = state + (int64_t)slots[s] * state_slot_stride + ((int64_t)h * V + col) * D;  // [H][V][D]
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = sub * R + r;
    S[r] = d < D ? column[d] : 0.f;
  }
  for (int i = 0; i < run.y; ++i) {
    const int64_t t = run.x + i;
    const float* kt = k + (t * G + g) * D;
    const float* qt = q + (t * G + g) * D;
    float kr[R], qr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = sub * R + r;
      kr[r] = d < D ? kt[d] : 0.f;
      qr[r] = d < D ? qt[d] : 0.f;
    }
    const float dec = channel_decay ? 0.f : decay[t * H + h], b = beta[t * H + h], vt = v[(t * H + h) * V + col];
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = sub * R + r;
      const float dr = channel_decay ? (d < D ? decay[(t * H + h) * D + d] : 0.f) : dec;
      S[r] = dr * S[r];
      dot = fmaf(S[r], kr[r], dot);
    }
    for (int off = L / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, L);
    const float u = delta ? b * (vt - dot) : b * vt;
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = fmaf(kr[r], u, S[r]);
      o = fmaf(S[r], qr[r], o);
    }
    for (int off = L / 2; off > 0; off >>= 1) o += __shfl_xor(o, off, L);
    if (sub == 0) out[(t * H + h) * V + col] = o;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = sub * R + r;
    if (d < D) column[d] = S[r];
  }
}

// The same recurrence for key widths up to 256, where the chain of dependent steps sets the time.  A
// column is owned by a group of L = 4, 8 or 16 neighbouring lanes, whose sums are added by cross-lane
// moves inside the register file (no trip through LDS); a lane holds R = D / L rows of its column
// (rows 4 L i + 4 sub .. + 3, so that a group's reads of k and q are contiguous).  The wider the keys,
// the more lanes share a column, which keeps the chain of a step short: 4 R multiply-adds and two
// sums over the group.  A workgroup has 16 columns (16 L threads); the step's inputs reach it
// through LDS in chunks of CH tokens, the next chunk being fetched from memory into registers while
// the current one is worked through, so no step waits for memory.
template <int L>
__device__ __forceinline__ float group_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));  // lanes (1, 0, 3, 2) of a quad
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));  // lanes (2, 3, 0, 1)
  if (L >= 8) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));   // 8 lanes mirrored
  if (L >= 16) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));  // 16 lanes mirrored
  return v;
}

template <int R, int L, int CH, bool CHANNEL, bool DELTA>
__global__ __launch_bounds__(16 * L) void delta_recurrence_group_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ beta,
    const float* __restrict__ decay, const int4* __restrict__ seq_runs, const int* __restrict__ slots,
    float* __restrict__ state, int64_t state_slot_stride, int G, int H, int D, int V, float* __restrict__ out) {
  constexpr int NT = 16 * L;         // threads: 16 columns of L lanes
  constexpr int DP = L * R;          // rows of a column, padded
  constexpr int KQ = CH * DP / NT;   // numbers of k (and of q) a thread fetches per chunk
  constexpr int VN = CH * 16 / NT;   // of v
  static_assert(R % 4 == 0 && CH * DP % (4 * NT) == 0 && CH * 16 % NT == 0 && 2 * CH <= NT, "chunk shape");
  __shared__ __attribute__((aligned(16))) float s_k[CH * DP];
  __shared__ __attribute__((aligned(16))) float s_q[CH * DP];
  __shared__ __attribute__((aligned(16))) float s_dec[CHANNEL ? CH * DP : 4];  // a decay per key channel
  __shared__ float s_v[CH * 16];
  __shared__ float s_bd[2 * CH];     // beta, then decay (one per head)
  const int s = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * 16;
  const int tid = threadIdx.x;
  const int col = col0 + tid / L, sub = tid % L;
  const bool live = col < V;
  const int4 run = seq_runs[s];
  const int g = h / (H / G);
  float* column = state + (int64_t)slots[s] * state_slot_stride + ((int64_t)h * V + (live ? col : 0)) * D;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = (r >> 2) * (4 * L) + sub * 4 + (r & 3);
    S[r] = (live && d < D) ? column[d] : 0.f;
  }
  const bool vec = D % 4 == 0;
  float pk[KQ], pq[KQ], pd[CHANNEL ? KQ : 1], pv[VN], pbd;
  // a thread's share of the chunk that starts at token `first` of the run, from memory into registers
  auto fetch = [&](int first) {
    if (vec) {
#pragma unroll
      for (int p = 0; p < KQ / 4; ++p) {
        const int e = (tid + NT * p) * 4, i = e / DP, d = e % DP;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
        if (first + i < run.y && d < D) {
          const int64_t at = ((int64_t)(run.x + first + i) * G + g) * D + d;
          a = *reinterpret_cast<const float4*>(k + at);
          b = *reinterpret_cast<const float4*>(q + at);
        }
        pk[4 * p] = a.x; pk[4 * p + 1] = a.y; pk[4 * p + 2] = a.z; pk[4 * p + 3] = a.w;
        pq[4 * p] = b.x; pq[4 * p + 1] = b.y; pq[4 * p + 2] = b.z; pq[4 * p + 3] = b.w;
        if (CHANNEL) {
          float4 c = make_float4(0.f, 0.f, 0.f, 0.f);
          if (first + i < run.y && d < D)
            c = *reinterpret_cast<const float4*>(decay + ((int64_t)(run.x + first + i) * H + h) * D + d);
          pd[4 * p] = c.x; pd[4 * p + 1] = c.y; pd[4 * p + 2] = c.z; pd[4 * p + 3] = c.w;
        }
      }
    } else {
#pragma unroll
      for (int p = 0; p < KQ; ++p) {
        const int e = tid + NT * p, i = e / DP, d = e % DP;
        const bool there = first + i < run.y && d < D;
        const int64_t at = ((int64_t)(run.x + first + i) * G + g) * D + d;
        pk[p] = there ? k[at] : 0.f;
        pq[p] = there ? q[at] : 0.f;
        if (CHANNEL) pd[p] = there ? decay[((int64_t)(run.x + first + i) * H + h) * D + d] : 0.f;
      }
    }
#pragma unroll
    for (int p = 0; p < VN; ++p) {
      const int e = tid + NT * p, i = e / 16, c = col0 + e % 16;
      pv[p] = (first + i < run.y && c < V) ? v[((int64_t)(run.x + first + i) * H + h) * V + c] : 0.f;
    }
    pbd = 0.f;
    if (tid < (CHANNEL ? CH : 2 * CH) && first + tid % CH < run.y)
      pbd = (tid < CH ? beta : decay)[(int64_t)(run.x + first + tid % CH) * H + h];
  };
  auto stage = [&]() {
    if (vec) {
#pragma unroll
      for (int p = 0; p < KQ / 4; ++p) {
        const int e = (tid + NT * p) * 4;
        *reinterpret_cast<float4*>(s_k + e) = make_float4(pk[4 * p], pk[4 * p + 1], pk[4 * p + 2], pk[4 * p + 3]);
        *reinterpret_cast<float4*>(s_q + e) = make_float4(pq[4 * p], pq[4 * p + 1], pq[4 * p + 2], pq[4 * p + 3]);
        if (CHANNEL) *reinterpret_cast<float4*>(s_dec + e) = make_float4(pd[4 * p], pd[4 * p + 1], pd[4 * p + 2], pd[4 * p + 3]);
      }
    } else {
#pragma unroll
      for (int p = 0; p < KQ; ++p) {
        s_k[tid + NT * p] = pk[p];
        s_q[tid + NT * p] = pq[p];
        if (CHANNEL) s_dec[tid + NT * p] = pd[p];
      }
    }
#pragma unroll
    for (int p = 0; p < VN; ++p) s_v[tid + NT * p] = pv[p];
    if (tid < 2 * CH) s_bd[tid] = pbd;
  };
  fetch(0);
  for (int first = 0; first < run.y; first += CH) {
    __syncthreads();  // the chunk before has been worked through
    stage();
    __syncthreads();
    if (first + CH < run.y) fetch(first + CH);
    const int n = min(CH, run.y - first);
    for (int i = 0; i < n; ++i) {
      const float* kt = s_k + i * DP;
      const float* qt = s_q + i * DP;
      const float dec = s_bd[CH + i], b = s_bd[i], vt = s_v[i * 16 + tid / L];
      float kr[R];
      float dot = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 k4 = *reinterpret_cast<const float4*>(kt + r4 * (4 * L) + sub * 4);
        kr[4 * r4] = k4.x; kr[4 * r4 + 1] = k4.y; kr[4 * r4 + 2] = k4.z; kr[4 * r4 + 3] = k4.w;
      }
      if (CHANNEL) {
#pragma unroll
        for (int r4 = 0; r4 < R / 4; ++r4) {
          const float4 d4 = *reinterpret_cast<const float4*>(s_dec + i * DP + r4 * (4 * L) + sub * 4);
          S[4 * r4] *= d4.x; S[4 * r4 + 1] *= d4.y; S[4 * r4 + 2] *= d4.z; S[4 * r4 + 3] *= d4.w;
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) S[r] = dec * S[r];
      }
      if (DELTA) {
#pragma unroll
        for (int r = 0; r < R; ++r) dot = fmaf(S[r], kr[r], dot);
        dot = group_sum<L>(dot);
      }
      const float u = DELTA ? b * (vt - dot) : b * vt;
      float o = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 q4 = *reinterpret_cast<const float4*>(qt + r4 * (4 * L) + sub * 4);
        S[4 * r4 + 0] = fmaf(kr[4 * r4 + 0], u, S[4 * r4 + 0]); o = fmaf(S[4 * r4 + 0], q4.x, o);
        S[4 * r4 + 1] = fmaf(kr[4 * r4 + 1], u, S[4 * r4 + 1]); o = fmaf(S[4 * r4 + 1], q4.y, o);
        S[4 * r4 + 2] = fmaf(kr[4 * r4 + 2], u, S[4 * r4 + 2]); o = fmaf(S[4 * r4 + 2], q4.z, o);
        S[4 * r4 + 3] = fmaf(kr[4 * r4 + 3], u, S[4 * r4 + 3]); o = fmaf(S[4 * r4 + 3], q4.w, o);
      }
      o = group_sum<L>(o);
      if (live && sub == 0) out[((int64_t)(run.x + first + i) * H + h) * V + col] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = (r >> 2) * (4 * L) + sub * 4 + (r & 3);
      if (d < D) column[d] = S[r];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(PAE_WAVE) void delta_gated_norm_kernel(const float* __restrict__ o, const T* __restrict__ gates,
                                                                    int64_t gate_stride, int gate_sigmoid,
                                                                    const void* __restrict__ weight, int w_is_f32, float eps,
                                                                    int H, int V, T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + (t * H + h) * V;
  float ss = 0.f;
  for (int i = lane; i < V; i += PAE_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + eps);
  const T* gate = gates + t * gate_stride + h * V;
  for (int i = lane; i < V; i += PAE_WAVE) {
    const float z = to_f32(gate[i]);
    const float gz = gate_sigmoid ? 1.0f / (1.0f + expf(-z)) : silu_f(z);
    out[(t * H + h) * V + i] = from_f32<T>(x[i] * inv * load_param(weight, w_is_f32, i) * gz);
  }
}

// The gated norm over a step's read-outs `o` [T][H][V], for mixers that share it (linear_attention.hip).
int pae_launch_gated_norm(int dtype, const float* o, const void* gates, int64_t gate_stride, int gate_sigmoid,
                          const void* weight, int w_is_f32, float eps, int num_tokens, int H, int V, void* out,
                          hipStream_t stream) {
  dim3 grid(num_tokens, H);
  if (dtype == PAE_F32)
    delta_gated_norm_kernel<float><<<grid, PAE_WAVE, 0, stream>>>(o, (const float*)gates, gate_stride, gate_sigmoid, weight,
                                                                  w_is_f32, eps, H, V, (float*)out);
  else if (dtype == PAE_BF16)
    delta_gated_norm_kernel<bf16_t><<<grid, PAE_WAVE, 0, stream>>>(o, (const bf16_t*)gates, gate_stride, gate_sigmoid, weight,
                                                                   w_is_f32, eps, H, V, (bf16_t*)out);
  else
    return pae_fail("gated norm: unknown dtype code %d", dtype);
  return 0;
}

static int lanes_per_column(int D, int R);
void pae_launch_recurrence(const float* q, const float* k, const float* v, const float* beta, const float* decay,
                           const int4* runs, const int* slots, float* state, int64_t state_slot_stride, int G, int H,
                           int D, int V, int num_seqs, int channel_decay, int delta, float* o, hipStream_t stream);

// The recurrence over a step's rows for every (sequence, head, column of S).  `channel_decay`: `decay` is
// [T][H][D] instead of [T][H]; `delta` off: u = beta v (a memory that only adds).
void pae_launch_recurrence(const float* q, const float* k, const float* v, const float* beta, const float* decay,
                           const int4* runs, const int* slots, float* state, int64_t state_slot_stride, int G, int H,
                           int D, int V, int num_seqs, int channel_decay, int delta, float* o, hipStream_t stream) {
  dim3 group_grid((V + 15) / 16, H, num_seqs);
  // (rows a lane, lanes a column, tokens a chunk)
#define GROUP_AS(R, L, CH, CHANNEL, DELTA)                                                                        \
  delta_recurrence_group_kernel<R, L, CH, CHANNEL, DELTA><<<group_grid, 16 * L, 0, stream>>>(                     \
      q, k, v, beta, decay, runs, slots, state, state_slot_stride, G, H, D, V, o)
#define GROUP(R, L, CH)                                       \
  do {                                                        \
    if (channel_decay && delta) GROUP_AS(R, L, CH, true, true);      \
    else if (channel_decay) GROUP_AS(R, L, CH, true, false);  \
    else if (delta) GROUP_AS(R, L, CH, false, true);          \
    else GROUP_AS(R, L, CH, false, false);                    \
  } while (0)
  if (D <= 16) GROUP(4, 4, 32);
  else if (D <= 32) GROUP(8, 4, 32);
  else if (D <= 64) GROUP(8, 8, 16);
  else if (D <= 128) GROUP(8, 16, 16);
  else if (D <= 256) GROUP(16, 16, 16);
  else {
    const int L = lanes_per_column(D, 16);
    dim3 rec_grid((V + 256 / L - 1) / (256 / L), H, num_seqs);
    delta_recurrence_kernel<16><<<rec_grid, 256, 0, stream>>>(q, k, v, beta, decay, runs, slots, state,
                                                              state_slot_stride, G, H, D, V, L, channel_decay, delta, o);
  }
#undef GROUP
#undef GROUP_AS
}

static int lanes_per_column(int D, int R) {
  int L = 1;
  while (L * R < D) L *= 2;
  return L;
}

static int64_t work_part(int64_t floats) { return (floats + 3) / 4 * 4; }

extern "C" int pae_delta_rule_step(int dtype, const void* proj, int64_t row_stride, int num_tokens, int num_seqs,
                                   const int* tok_seq, const int* positions, const int* seq_runs, const int* slots,
                                   const float* conv_w, float* conv_tail, int64_t tail_slot_stride, int taps, int G,
                                   int H, int D, int V, const float* a_log, const float* dt_bias, float unit_eps,
                                   float* state, int64_t state_slot_stride, const void* norm_w, int w_is_f32,
                                   float norm_eps, float* work, void* out, const void* gate_in, int64_t gate_stride,
                                   int gate_sigmoid, const void* b_in, int64_t b_stride, const void* a_in, int64_t a_stride,
                                   int channel_decay, hipStream_t stream) {
  PAE_REQUIRE(G > 0 && H > 0 && H % G == 0 && D > 0 && V > 0, "delta rule: bad head sizes G=%d H=%d D=%d V=%d", G, H, D, V);
  PAE_REQUIRE(taps >= 1 && taps <= 64, "delta rule: %d convolution taps", taps);
  PAE_REQUIRE(D <= 1024, "delta rule: key width %d exceeds 1024", D);
  PAE_REQUIRE(H <= 65535 && num_seqs <= 65535, "delta rule: %d heads, %d sequences exceed the grid", H, num_seqs);
  const int64_t C = 2 * (int64_t)G * D + (int64_t)H * V;
  PAE_REQUIRE(V <= 1024 && 2 * G + H <= 65535, "delta rule: value width %d or %d heads exceed the kernels' limits", V, 2 * G + H);
  PAE_REQUIRE(row_stride >= C, "delta rule: row stride %lld too small", (long long)row_stride);
  PAE_REQUIRE(gate_in && b_in && a_in, "delta rule: the gate's, beta's and the decay's rows are needed");
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "delta rule: unknown dtype code %d", dtype);
  if (num_tokens <= 0 || num_seqs <= 0) return 0;
  // work: q [T][G][D], k [T][G][D], v [T][H][V], beta [T][H], decay [T][H] or [T][H][D], o [T][H][V]
  // (every part starts on a 16-byte boundary: the recurrence reads k, q and channel decays four at a time)
  float* q = work;
  float* k = q + work_part((int64_t)num_tokens * G * D);
  float* v = k + work_part((int64_t)num_tokens * G * D);
  float* beta = v + work_part((int64_t)num_tokens * H * V);
  float* decay = beta + work_part((int64_t)num_tokens * H);
  float* o = decay + work_part((int64_t)num_tokens * H * (channel_decay ? D : 1));
  const int4* runs = (const int4*)seq_runs;
  dim3 tail_grid((unsigned)((C + 255) / 256), num_seqs);
  dim3 norm_grid(num_tokens, H);
#define DELTA_LAUNCH(T)                                                                                                 \
  delta_prepare_kernel<T><<<dim3(num_tokens, 2 * G + H), 128, 0, stream>>>(                                             \
      (const T*)proj, row_stride, tok_seq, positions, runs, slots, conv_w, conv_tail, tail_slot_stride, taps, G, H, D,  \
      V, a_log, dt_bias, unit_eps, (const T*)b_in, b_stride, (const T*)a_in, a_stride, channel_decay, q, k, v, beta,    \
      decay);                                                                                                           \
  if (taps > 1)                                                                                                         \
    delta_conv_tail_kernel<T><<<tail_grid, 256, 0, stream>>>((const T*)proj, row_stride, runs, slots, conv_tail,        \
                                                             tail_slot_stride, taps, (int)C);                           \
  pae_launch_recurrence(q, k, v, beta, decay, runs, slots, state, state_slot_stride, G, H, D, V, num_seqs,              \
                        channel_decay, 1, o, stream);                                                                   \
  delta_gated_norm_kernel<T><<<norm_grid, PAE_WAVE, 0, stream>>>(o, (const T*)gate_in, gate_stride, gate_sigmoid,       \
                                                                 norm_w, w_is_f32, norm_eps, H, V, (T*)out)
  if (dtype == PAE_F32) {
    DELTA_LAUNCH(float);
  } else {
    DELTA_LAUNCH(bf16_t);
  }
#undef DELTA_LAUNCH
  return pae_check_launch("delta_rule_step");
}

// floats of `work` that pae_delta_rule_step needs for a step of `num_tokens` rows
extern "C" int64_t pae_delta_rule_work_floats(int num_tokens, int G, int H, int D, int V, int channel_decay) {
  const int64_t T = num_tokens;
  return 2 * work_part(T * G * D) + 2 * work_part(T * H * V) + work_part(T * H) + work_part(T * H * (channel_decay ? D : 1));
}
