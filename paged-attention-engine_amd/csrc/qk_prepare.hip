// Query/key normalisation over the whole projection, rotation by position and the cache write,
// in one pass over a token's projected row.
//
// A row holds [q: nh heads of hd | k: nkv heads of hd | v: nkv heads of vd].  With `norm` set, the
// whole q part is divided by its root mean square (mean over all nh * hd features, eps inside the
// root) and multiplied by a weight of that size, and likewise the k part: one statistic per
// projection, not per head.  With `per_head` instead, every q head and every k head is divided by its own root
// mean square over hd and multiplied by a weight of hd numbers that the heads share.  Then the first `rot` features of every q and k head turn by the
// token's angles: pair i is (2i, 2i + 1) with `interleaved`, (i, i + rot / 2) without, and
//   (u, v) -> (u c - v s, v c + u s),  c = magnitude * cos(angle_i), s = magnitude * sin(angle_i)
// (a magnitude other than 1 is what frequency-scaled rotations multiply their tables by).
// Statistics, weights and the rotation are float32; a value is rounded to the storage type once,
// when it is written: queries in place, keys to [block][kv head][offset][hd], values transposed
// within the page, [block][kv head][vd][offset].
#include "common.h"
#include "api.h"

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rotate_store_kernel(
    T* __restrict__ qkv, int64_t row_stride, int nh, int nkv, int hd, int vd, const void* __restrict__ q_w,
    const void* __restrict__ k_w, int w_is_f32, float eps, int rot, int interleaved,
    const float* __restrict__ cos_sin, float magnitude, const int* __restrict__ positions,
    const int* __restrict__ tok_seq, const int* __restrict__ block_tables, int max_blocks, int bs,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int write_kv, int per_head) {
  extern __shared__ float head_inv[];  // [nh + nkv] with `per_head`
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  T* row = qkv + (int64_t)t * row_stride;
  const int nq = nh * hd, nk = nkv * hd;
  // the token's place in the cache is asked for first: the answer arrives while the sums are formed
  const int pos = positions[t];
  const int off = pos % bs;
  int64_t k_base = 0, v_base = 0;  // element offsets of (block, kv head 0) in the pools
  if (write_kv) {
    const int64_t block = block_tables[(int64_t)tok_seq[t] * max_blocks + pos / bs];
    k_base = block * nkv * (int64_t)bs * hd;
    v_base = block * nkv * (int64_t)bs * vd;
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (q_w && per_head) {
    // a wavefront a head in turn: its lanes share out the head's features, and meet in a fixed order
    const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
    for (int h = wave; h < nh + nkv; h += 4) {
      float ss = 0.f;
      for (int i = lane; i < hd; i += PAE_WAVE) { const float x = to_f32(row[h * hd + i]); ss = fmaf(x, x, ss); }
      ss = wave_sum(ss);
      if (lane == 0) head_inv[h] = 1.0f / sqrtf(ss / (float)hd + eps);
    }
    __syncthreads();
  } else if (q_w) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) { const float x = to_f32(row[i]); sq = fmaf(x, x, sq); }
    for (int i = threadIdx.x; i < nk; i += 256) { const float x = to_f32(row[nq + i]); sk = fmaf(x, x, sk); }
    sq = block_sum<4>(sq, scratch);
    inv_q = 1.0f / sqrtf(sq / (float)nq + eps);
    if (nk) {
      sk = block_sum<4>(sk, scratch);
      inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
    }
  }
  // feature j of the row (j < nq + nk), normalised
  auto at = [&](int j) {
    const float x = to_f32(row[j]);
    if (!q_w) return x;
    if (per_head) return x * head_inv[j / hd] * load_param(j < nq ? q_w : k_w, w_is_f32, j % hd);
    return j < nq ? x * inv_q * load_param(q_w, w_is_f32, j) : x * inv_k * load_param(k_w, w_is_f32, j - nq);
  };
  auto put = [&](int h, int i, float value) {  // head h (queries first, then keys), feature i
    if (h < nh) row[h * hd + i] = from_f32<T>(value);
    else k_cache[k_base + ((int64_t)(h - nh) * bs + off) * hd + i] = from_f32<T>(value);
  };
  const int half = rot / 2;
  const int heads = nh + (write_kv ? nkv : 0);
  for (int idx = threadIdx.x; idx < heads * half; idx += 256) {
    const int h = idx / half, i = idx % half;
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    const float c = magnitude * cos_sin[((int64_t)t * half + i) * 2], s = magnitude * cos_sin[((int64_t)t * half + i) * 2 + 1];
    const float a = at(h * hd + ia), b = at(h * hd + ib);
    put(h, ia, a * c - b * s);
    put(h, ib, b * c + a * s);
  }
  const int tail = hd - rot;  // features beyond the rotated ones: normalised (or copied) only
  if (q_w || write_kv)
    for (int idx = threadIdx.x; idx < heads * tail; idx += 256) {
      const int h = idx / tail, i = rot + idx % tail;
      if (h < nh && !q_w) continue;
      put(h, i, at(h * hd + i));
    }
  if (!write_kv) return;
  for (int idx = threadIdx.x; idx < nkv * vd; idx += 256) {
    const int h = idx / vd, i = idx % vd;
    v_cache[v_base + ((int64_t)h * vd + i) * bs + off] = row[nq + nk + idx];
  }
}

extern "C" int pae_qk_norm_rotate_store(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nh, int nkv,
                                        int hd, int vd, const void* q_w, const void* k_w, int w_is_f32, float eps,
                                        int rot, int interleaved, const float* cos_sin, float magnitude,
                                        const int* positions, const int* tok_seq, const int* block_tables,
                                        int max_blocks, int bs, void* k_cache, void* v_cache, int write_kv,
                                        int per_head, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && vd > 0, "qk_norm_rotate_store: bad head sizes nh=%d nkv=%d hd=%d vd=%d",
              nh, nkv, hd, vd);
  PAE_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "qk_norm_rotate_store: %d rotated features of %d", rot, hd);
  PAE_REQUIRE(rot == 0 || cos_sin, "qk_norm_rotate_store: a rotation needs its table of cosines and sines");
  PAE_REQUIRE((q_w == nullptr) == (k_w == nullptr) || nkv == 0, "qk_norm_rotate_store: one norm weight without the other");
  PAE_REQUIRE(row_stride >= (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd, "qk_norm_rotate_store: row stride %lld too small",
              (long long)row_stride);
  PAE_REQUIRE(!write_kv || (nkv > 0 && bs > 0 && max_blocks > 0 && k_cache && v_cache && block_tables && tok_seq),
              "qk_norm_rotate_store: a cache write needs tables and pools");
  if (num_tokens <= 0) return 0;
  const size_t lds = per_head ? (size_t)(nh + nkv) * sizeof(float) : 0;
  PAE_REQUIRE(lds <= 32768, "qk_norm_rotate_store: %d heads with norms of their own", nh + nkv);
  if (dtype == PAE_F32)
    qk_norm_rotate_store_kernel<float><<<num_tokens, 256, lds, stream>>>(
        (float*)qkv, row_stride, nh, nkv, hd, vd, q_w, k_w, w_is_f32, eps, rot, interleaved, cos_sin, magnitude,
        positions, tok_seq, block_tables, max_blocks, bs, (float*)k_cache, (float*)v_cache, write_kv, per_head);
  else if (dtype == PAE_BF16)
    qk_norm_rotate_store_kernel<bf16_t><<<num_tokens, 256, lds, stream>>>(
        (bf16_t*)qkv, row_stride, nh, nkv, hd, vd, q_w, k_w, w_is_f32, eps, rot, interleaved, cos_sin, magnitude,
        positions, tok_seq, block_tables, max_blocks, bs, (bf16_t*)k_cache, (bf16_t*)v_cache, write_kv, per_head);
  else
    return pae_fail("qk_norm_rotate_store: unknown dtype code %d", dtype);
  return pae_check_launch("qk_norm_rotate_store");
}
