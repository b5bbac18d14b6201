// Latent attention over the paged cache on the matrix cores (bfloat16 in, float32 scores, softmax
// and accumulation): every head of a token scores the same cached row (latent + rotated key part,
// KD wide) and sums the rows' first C features as its values.
//
// The cache holds the rows twice: `latent` [block][page][KD], a key per row, and `latent_t`
// [block][C][page], the same latents transposed within the page, which is the layout the second
// product's operand wants (see attention_mfma.hip: S^T = K Q^T, O^T += V^T P^T, the scores' accumulator
// layout being the second product's B operand).  A "column" is one (token, head); a workgroup takes
// 16 CT columns, the heads of one or several consecutive tokens of a sequence (head fastest), and one
// slice of VS value features; its four wavefronts take the 16-key tiles in turn and merge through LDS.
// All heads share the keys, so a tile of keys is read once for all of a workgroup's columns; the slices
// of the values repeat the scores (18 matrix instructions a tile at KD = 576) to keep the output tile
// (VS / 16 accumulators a column tile) and the queries (KD / 32 operands a column tile) in registers.
//
// Mask: position p sees the keys first_visible(p) .. p: a sliding window (p - window + 1 on), chunks
// (p - p % window on), or every earlier key (window 0).  A column's result depends on its own position
// alone: keys outside add exact zeros, pages that a window has passed (table entry -1) are not read.
#include "common.h"
#include "api.h"
#include "attention_device.h"

__device__ __forceinline__ int latent_first_visible(int pos, int window, int chunked) {
  if (window <= 0) return 0;
  if (chunked) return pos - pos % window;
  return pos - window + 1 > 0 ? pos - window + 1 : 0;
}

// tiles[i] = (table row of the sequence, first flat token, tokens, unused); blockIdx = (tile, value slice, head group)
template <int KD, int VS, int CT>
__global__ __launch_bounds__(256, 1) void latent_attn_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ latent, const bf16_t* __restrict__ latent_t, const int4* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks, int bs, int H, int C,
    float scale_log2, int window, int chunked, int num_splits, int split_len, float* __restrict__ part_acc,
    float* __restrict__ part_ml, const float* __restrict__ sinks) {
  extern __shared__ float s_buf[];  // [3 or 1][CT][VS / 4 + 2][64]
  constexpr int ROWS = VS / 4 + 2;
  const int lane = threadIdx.x % PAE_WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE);
  const int col = lane % 16, g4 = lane / 16;
  // with splits (single tokens with long contexts): workgroup (tile, split) takes the keys
  // [split * split_len, + split_len) and leaves unnormalised sums for the merge kernel
  const int tile_index = blockIdx.x / num_splits, split = blockIdx.x % num_splits;
  const int4 tile = tiles[tile_index];
  const int slice = blockIdx.y, head0 = blockIdx.z * 16;
  const int hpg = H - head0 < 16 ? H - head0 : 16;  // heads of this group
  const int* table = block_tables + (int64_t)tile.x * max_blocks;
  const int tok0 = tile.y, ntok = tile.z;
  const int pos0 = positions[tok0];

  int pos[CT], start[CT], tok[CT], head[CT];
  bf16x8 qf[CT][KD / 32];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + col;
    const int t = c / hpg;
    const bool live = t < ntok;
    tok[ct] = tok0 + (live ? t : 0);
    head[ct] = head0 + c % hpg;
    pos[ct] = live ? pos0 + t : -1;  // a dead column sees no key
    start[ct] = live ? latent_first_visible(pos[ct], window, chunked) : 0;
    const bf16_t* qrow = q + (int64_t)tok[ct] * q_stride + (int64_t)head[ct] * KD;
#pragma unroll
    for (int j = 0; j < KD / 32; ++j) qf[ct][j] = *reinterpret_cast<const bf16x8*>(qrow + 32 * j + 8 * g4);
  }
  int hi = pos0 + ntok - 1;
  int lo = latent_first_visible(pos0, window, chunked) / 16 * 16;
  if (num_splits > 1) {
    lo = max(lo, split * split_len);
    hi = min(hi, (split + 1) * split_len - 1);
    if (lo > hi) return;  // the merge kernel knows which splits hold keys
  }

  f32x4 acc[CT][VS / 16];
  float m[CT], l[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    m[ct] = NEG_BIG;
    l[ct] = 0.f;
#pragma unroll
    for (int t = 0; t < VS / 16; ++t) acc[ct][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  const int lrow = lane / 4, lgrp = lane % 4;
  // Two register sets of keys and values take turns: the next tile's loads are in flight while this tile's
  // products run (a wavefront walks its tiles alone, with no other wavefront of its own to hide the wait).
  bf16x8 kfa[KD / 32], kfb[KD / 32];
  s16x4 vfa[VS / 16], vfb[VS / 16];
  auto load = [&](bf16x8 (&kf)[KD / 32], s16x4 (&vf)[VS / 16], int key0) {
    const int64_t block = max(table[key0 / bs], 0);  // a page the window has passed: all its keys are masked
    const bf16_t* kp = latent + (block * bs + key0 % bs) * (int64_t)KD;
    const bf16_t* vp = latent_t + (block * C + (int64_t)slice * VS) * bs + key0 % bs;
#pragma unroll
    for (int j = 0; j < KD / 32; ++j) kf[j] = *reinterpret_cast<const bf16x8*>(kp + lrow * KD + 32 * j + 8 * lgrp);
#pragma unroll
    for (int t = 0; t < VS / 16; ++t)
      vf[t] = *reinterpret_cast<const s16x4*>(vp + (int64_t)(16 * t + col) * bs + 4 * g4);
  };
  auto compute = [&](bf16x8 (&kf)[KD / 32], s16x4 (&vf)[VS / 16], int key0) {
    keys_to_mfma_order<KD>(kf);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KD / 32; ++j) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j], qf[ct][j], s, 0, 0, 0);
      float mx = NEG_BIG;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 4 * g4 + i;
        s[i] = (key <= pos[ct] && key >= start[ct]) ? s[i] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, s[i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, PAE_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, PAE_WAVE));
      const float m_new = fmaxf(m[ct], mx);
      const float alpha = exp2f(m[ct] - m_new);
      m[ct] = m_new;
      float psum = 0.f;
      s16x4 pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = exp2f(s[i] - m_new);
        psum += p;
        pb[i] = bf16_bits(p);
      }
      l[ct] = l[ct] * alpha + psum;
      // the output tile is rescaled only if some column's maximum rose (a product with 1 changes nothing, so the
      // result is the same bit for bit; after the first tiles most tiles raise no maximum)
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int t = 0; t < VS / 16; ++t) acc[ct][t] *= alpha;
      }
#pragma unroll
      for (int t = 0; t < VS / 16; ++t)
        acc[ct][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[t], pb, acc[ct][t], 0, 0, 0);
    }
  };
  int key0 = lo + 16 * wave;  // the same in every lane of a wavefront: the branches on it are uniform
  if (key0 <= hi) {
    load(kfa, vfa, key0);
    while (true) {
      const bool more_b = key0 + 64 <= hi;
      if (more_b) load(kfb, vfb, key0 + 64);
      compute(kfa, vfa, key0);
      if (!more_b) break;
      const bool more_a = key0 + 128 <= hi;
      if (more_a) load(kfa, vfa, key0 + 128);
      compute(kfb, vfb, key0 + 64);
      if (!more_a) break;
      key0 += 128;
    }
  }

  // wavefronts 1..3 hand their state to wavefront 0 through LDS, one after the other (one wavefront's state at a
  // time keeps the buffer small: 33 KB at 512 value features); a lane holds the same (column, features) everywhere
  // (where three states fit 64 KB, which they do at the sizes built, they are written at once, into places of their own, and merged after one barrier)
  constexpr bool AT_ONCE = 3 * CT * ROWS * PAE_WAVE * sizeof(float) <= 64 * 1024;
  for (int w = 1; w < 4; ++w) {
    if (AT_ONCE ? (w == 1 && wave > 0) : wave == w) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        float* mine = s_buf + ((AT_ONCE ? wave - 1 : 0) * CT + ct) * ROWS * PAE_WAVE;
#pragma unroll
        for (int t = 0; t < VS / 16; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[(4 * t + i) * PAE_WAVE + lane] = acc[ct][t][i];
        mine[(VS / 4) * PAE_WAVE + lane] = m[ct];
        mine[(VS / 4 + 1) * PAE_WAVE + lane] = l[ct];
      }
    }
    if (!AT_ONCE || w == 1) __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const float* theirs = s_buf + ((AT_ONCE ? w - 1 : 0) * CT + ct) * ROWS * PAE_WAVE;
        const float mw = theirs[(VS / 4) * PAE_WAVE + lane];
        const float m_new = fmaxf(m[ct], mw);
        const float f0 = exp2f(m[ct] - m_new), fw = exp2f(mw - m_new);
#pragma unroll
        for (int t = 0; t < VS / 16; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[ct][t][i] = acc[ct][t][i] * f0 + theirs[(4 * t + i) * PAE_WAVE + lane] * fw;
        l[ct] = l[ct] * f0 + theirs[(VS / 4 + 1) * PAE_WAVE + lane] * fw;
        m[ct] = m_new;
      }
    }
    if (!AT_ONCE) __syncthreads();
  }
  if (wave != 0) return;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float sum = l[ct];
    sum += __shfl_xor(sum, 16, PAE_WAVE);
    sum += __shfl_xor(sum, 32, PAE_WAVE);
    if (pos[ct] < 0) continue;
    if (num_splits > 1) {  // CT is 1 here and the tile one token: partials by (tile, split, head)
      const int64_t slot = ((int64_t)tile_index * num_splits + split) * H + head[ct];
#pragma unroll
      for (int t = 0; t < VS / 16; ++t)
        *reinterpret_cast<f32x4*>(part_acc + slot * C + (int64_t)slice * VS + 16 * t + 4 * g4) = acc[ct][t];
      if (slice == 0 && g4 == 0) {
        part_ml[slot * 2] = m[ct];
        part_ml[slot * 2 + 1] = sum;
      }
      continue;
    }
    // a sink joins the denominator as exp(sink), unscaled, with no key and no value
    if (sinks) sum += exp2f(sinks[head[ct]] * LOG2E - m[ct]);
    const float inv = 1.0f / sum;
    bf16_t* o = out + (int64_t)tok[ct] * out_stride + (int64_t)head[ct] * C + (int64_t)slice * VS;
#pragma unroll
    for (int t = 0; t < VS / 16; ++t) {
      s16x4 w4;
#pragma unroll
      for (int i = 0; i < 4; ++i) w4[i] = bf16_bits(acc[ct][t][i] * inv);
      *reinterpret_cast<s16x4*>(o + 16 * t + 4 * g4) = w4;
    }
  }
}

// Adds a single token's partials in split order and writes the output: one workgroup per (tile, head), a thread
// per four features.
__global__ void latent_attn_merge_kernel(bf16_t* __restrict__ out, int64_t out_stride, const float* __restrict__ part_acc,
                                         const float* __restrict__ part_ml, const int4* __restrict__ tiles,
                                         const int* __restrict__ positions, int H, int C, int window, int chunked,
                                         int num_splits, int split_len, const float* __restrict__ sinks) {
  const int4 tile = tiles[blockIdx.x];
  const int head = blockIdx.y, tok = tile.y;
  const int pos = positions[tok];
  const int s_first = latent_first_visible(pos, window, chunked) / 16 * 16 / split_len, s_last = pos / split_len;
  const int d = threadIdx.x * 4;
  if (d >= C) return;
  float m = NEG_BIG, l = 0.f;
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
  for (int sp = s_first; sp <= s_last; ++sp) {
    const int64_t slot = ((int64_t)blockIdx.x * num_splits + sp) * H + head;
    const float ms = part_ml[slot * 2], ls = part_ml[slot * 2 + 1];
    const f32x4 v = *reinterpret_cast<const f32x4*>(part_acc + slot * C + d);
    const float m_new = fmaxf(m, ms);
    const float f_old = exp2f(m - m_new), f = exp2f(ms - m_new);
    a = a * f_old + v * f;
    l = l * f_old + ls * f;
    m = m_new;
  }
  if (sinks) l += exp2f(sinks[head] * LOG2E - m);
  const float inv = 1.0f / l;
  s16x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = bf16_bits(a[i] * inv);
  *reinterpret_cast<s16x4*>(out + (int64_t)tok * out_stride + (int64_t)head * C + d) = w;
}

#define LATENT_SPLIT_MAX_GROUPS 128  // unsplit workgroups up to which single tokens' keys are split
#define LATENT_SPLIT 256  // keys per split of a single token's attention (fixed: a result does not depend on the batch)
extern "C" int pae_latent_attn_split() { return LATENT_SPLIT; }

static size_t latent_lds_bytes(int ct, int vs) {  // three wavefronts' states if they fit 64 KB, else one
  const size_t one = (size_t)ct * (vs / 4 + 2) * PAE_WAVE * sizeof(float);
  return 3 * one <= 64 * 1024 ? 3 * one : one;
}

// Key widths (latent + rotated part) the kernel is built for; the value slice is the largest of 128, 64, 32 that divides C.
extern "C" int pae_latent_attn_supported(int kd, int C, int bs) {
  const bool kd_ok = kd == 64 || kd == 96 || kd == 128 || kd == 160 || kd == 192 || kd == 256 || kd == 288 || kd == 320 ||
                     kd == 384 || kd == 512 || kd == 576;
  return kd_ok && C % 32 == 0 && C > 0 && C <= kd && bs >= 16 && bs % 16 == 0;
}

extern "C" int pae_latent_attn_columns(int H, int ct) {  // tokens a tile of 16 ct columns holds
  const int hpg = H < 16 ? H : 16;
  return 16 * ct / hpg;
}

// `tiles` int32 [num_tiles][4]; ct = 1 (single tokens) or 2 (runs of tokens: tiles of up to pae_latent_attn_columns(H, 2) tokens).
extern "C" int pae_latent_attn_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* latent,
                                    const void* latent_t, const int* tiles, int num_tiles, int ct, const int* positions,
                                    const int* block_tables, int max_blocks, int bs, int H, int kd, int C, float scale,
                                    int window, int chunked, float* part_acc, float* part_ml, const float* sinks,
                                    hipStream_t stream) {
  PAE_REQUIRE(pae_latent_attn_supported(kd, C, bs), "latent attention: row width %d / latent %d / page size %d are not built", kd, C,
              bs);
  PAE_REQUIRE(H > 0 && H <= 16 * 65535 && max_blocks > 0 && window >= 0, "latent attention: bad sizes H=%d max_blocks=%d window=%d",
              H, max_blocks, window);
  PAE_REQUIRE(ct == 1 || ct == 2, "latent attention: %d column tiles a workgroup (1 or 2)", ct);
  PAE_REQUIRE(out_stride >= (int64_t)H * C && q_stride >= (int64_t)H * kd, "latent attention: row strides too small");
  if (num_tiles <= 0) return 0;
  const int vs = C % 128 == 0 ? 128 : (C % 64 == 0 ? 64 : 32);
  // Single tokens: the keys are split over workgroups when the tables reach beyond one split and the caller gave room
  // for the partial sums (num_tiles * splits * H * (C + 2) floats, splits = ceil(max_blocks * bs / pae_latent_attn_split())).
  int num_splits = 1;
  if (ct == 1 && part_acc && part_ml) num_splits = (int)(((int64_t)max_blocks * bs + LATENT_SPLIT - 1) / LATENT_SPLIT);
  // ... and only while the unsplit workgroups would leave most of the chip idle (measured at 576-wide rows, 12 heads,
  // context 4,096: one token 146 us unsplit, 15 + 8 us split and merged; 8 tokens 150 and 43 + 8; 32 tokens split 152;
  // 64 tokens unsplit 175).  The choice moves a result by the order of adding alone.
  if ((int64_t)num_tiles * (C / vs) * ((H + 15) / 16) > LATENT_SPLIT_MAX_GROUPS) num_splits = 1;
  PAE_REQUIRE((int64_t)num_tiles * num_splits <= 0x7fffffff, "latent attention: %d tiles of %d splits exceed the grid", num_tiles,
              num_splits);
  PAE_REQUIRE(num_splits == 1 || C / 4 <= 1024, "latent attention: latent %d too wide for the merge", C);
  dim3 grid(num_tiles * num_splits, C / vs, (H + 15) / 16);
  const float scale_log2 = scale * LOG2E;
#define LAT_LAUNCH(KD, VS, CT)                                                                                          \
  latent_attn_kernel<KD, VS, CT><<<grid, 256, latent_lds_bytes(CT, VS), stream>>>(                                       \
      (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)latent, (const bf16_t*)latent_t,             \
      (const int4*)tiles, positions, block_tables, max_blocks, bs, H, C, scale_log2, window, chunked, num_splits,       \
      LATENT_SPLIT, part_acc, part_ml, sinks)
#define LAT_BY_CT(KD, VS)        \
  if (ct == 1) {                 \
    LAT_LAUNCH(KD, VS, 1);       \
  } else {                       \
    LAT_LAUNCH(KD, VS, 2);       \
  }
#define LAT_BY_VS(KD)            \
  if (vs == 128) {               \
    LAT_BY_CT(KD, 128);          \
  } else if (vs == 64) {         \
    LAT_BY_CT(KD, 64);           \
  } else {                       \
    LAT_BY_CT(KD, 32);           \
  }
  switch (kd) {
    case 64: LAT_BY_VS(64); break;
    case 96: LAT_BY_VS(96); break;
    case 128: LAT_BY_VS(128); break;
    case 160: LAT_BY_VS(160); break;
    case 192: LAT_BY_VS(192); break;
    case 256: LAT_BY_VS(256); break;
    case 288: LAT_BY_VS(288); break;
    case 320: LAT_BY_VS(320); break;
    case 384: LAT_BY_VS(384); break;
    case 512: LAT_BY_VS(512); break;
    case 576: LAT_BY_VS(576); break;
    default: return pae_fail("latent attention: row width %d is not built", kd);
  }
#undef LAT_BY_VS
#undef LAT_BY_CT
#undef LAT_LAUNCH
  if (num_splits > 1) {
    const int threads = (C / 4 + PAE_WAVE - 1) / PAE_WAVE * PAE_WAVE;
    latent_attn_merge_kernel<<<dim3(num_tiles, H), threads, 0, stream>>>((bf16_t*)out, out_stride, part_acc, part_ml,
                                                                       (const int4*)tiles, positions, H, C, window, chunked,
                                                                       num_splits, LATENT_SPLIT, sinks);
  }
  return pae_check_launch("latent_attn");
}
