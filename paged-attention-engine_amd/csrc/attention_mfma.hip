// Causal attention over the paged cache on the matrix cores (bfloat16 in,
// float32 scores, softmax and accumulation).
//
// Both kernels work on transposed tiles so that the softmax output can feed the
// second product without leaving registers:
//   S^T[16 keys x 16 columns] = K[16 keys x hd] * Q^T        (MFMA 16x16x32, k = hd)
//   O^T[hd x 16 columns]     += V^T[hd x 16 keys] * P^T       (MFMA 16x16x16, k = keys)
// The accumulator layout of S^T (lane = column, registers = 4 consecutive keys) is
// exactly the B-operand layout of the second product.  A "column" is one (token,
// query head); the 16 keys of a tile are one cache page (or a 16-key slice of a
// larger page).  Keys live as [block][kv head][page][hd], values transposed as
// [block][kv head][hd][page], so both A operands are contiguous per lane.
//
// decode:  one workgroup per (sequence with a single new token, kv head, split of
//          the keys); the columns are the query heads that share the kv head, so a
//          page is read once for all of them.  Four wavefronts take pages in turn
//          and merge in LDS; the last workgroup to finish merges the splits.  Splits
//          start at multiples of the split length from position 0.
// prefill: one wavefront per (32 consecutive tokens of a sequence, query head).
//
// Masking is the reference's rule (engine/attention.py:474-487: key j visible iff
// j <= position of the query) plus an optional window.  A column's result depends
// only on its own position: fully masked pages add exact zeros.
#include "common.h"
#include "api.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;

#define NEG_BIG (-1.0e30f)
#define LOG2E 1.4426950408889634f

__device__ __forceinline__ short bf16_bits(float x) {
  const bf16_t h = __float2bfloat16(x);
  return *reinterpret_cast<const short*>(&h);
}

// State of CT column tiles of one wavefront.
template <int HD, int CT>
struct AttnState {
  f32x4 acc[CT][HD / 16];  // O^T: rows hd = 16 t + 4 g4 + i, column = lane % 16
  float m[CT];             // running maximum of the column (in units of log2)
  float l[CT];             // this lane's share of the column's sum
};

// One 16-key tile.  `kp` points at key row 0 of the tile (row stride HD), `vp` at
// value feature 0 of the tile's first key (feature stride `vstride` elements).
// q[ct][j]: B operand of column tile ct for hd slice j.  pos/start: per lane's column.
template <int HD, int CT>
__device__ __forceinline__ void attn_tile(AttnState<HD, CT>& st, const bf16x8 (&kf)[HD / 32],
                                          const s16x4 (&vf)[HD / 16], const bf16x8 (&q)[CT][HD / 32],
                                          int key0, const int (&pos)[CT], const int (&start)[CT],
                                          float scale_log2) {
  const int g4 = threadIdx.x % PAE_WAVE / 16;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j], q[ct][j], s, 0, 0, 0);
    float mx = NEG_BIG;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + 4 * g4 + i;
      s[i] = (key <= pos[ct] && key >= start[ct]) ? s[i] * scale_log2 : -INFINITY;
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, PAE_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, PAE_WAVE));
    const float m_new = fmaxf(st.m[ct], mx);
    const float alpha = exp2f(st.m[ct] - m_new);
    st.m[ct] = m_new;
    float psum = 0.f;
    s16x4 pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = exp2f(s[i] - m_new);
      psum += p;
      pb[i] = bf16_bits(p);
    }
    st.l[ct] = st.l[ct] * alpha + psum;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) {
      st.acc[ct][t] *= alpha;
      st.acc[ct][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[t], pb, st.acc[ct][t], 0, 0, 0);
    }
  }
}

// Loads are made with the lane order (row = lane / 4, group = lane % 4), so that the four lanes of
// a quad read contiguous bytes (64 of a key row, 32 of a value row) and the memory pipeline sees
// one access for them; `kv_to_mfma_order` then moves every register to the order the matrix
// instruction wants (row = lane % 16, group = lane / 16) with one cross-lane permute each.
template <int HD>
__device__ __forceinline__ void load_kv_tile(bf16x8 (&kf)[HD / 32], s16x4 (&vf)[HD / 16], const bf16_t* kp,
                                             const bf16_t* vp, int vstride) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int r = lane / 4, g = lane % 4;
#pragma unroll
  for (int j = 0; j < HD / 32; ++j) kf[j] = *reinterpret_cast<const bf16x8*>(kp + r * HD + 32 * j + 8 * g);
#pragma unroll
  for (int t = 0; t < HD / 16; ++t)
    vf[t] = *reinterpret_cast<const s16x4*>(vp + (int64_t)(16 * t + r) * vstride + 4 * g);
}

template <int HD>
__device__ __forceinline__ void kv_to_mfma_order(bf16x8 (&kf)[HD / 32], s16x4 (&vf)[HD / 16]) {
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  typedef __attribute__((ext_vector_type(2))) int i32x2;
  const int lane = threadIdx.x % PAE_WAVE;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;  // byte address of the source lane
#pragma unroll
  for (int j = 0; j < HD / 32; ++j) {
    i32x4 raw = *reinterpret_cast<i32x4*>(&kf[j]);
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = __builtin_amdgcn_ds_bpermute(fetch_from, raw[i]);
    kf[j] = *reinterpret_cast<bf16x8*>(&raw);
  }
#pragma unroll
  for (int t = 0; t < HD / 16; ++t) {
    i32x2 raw = *reinterpret_cast<i32x2*>(&vf[t]);
#pragma unroll
    for (int i = 0; i < 2; ++i) raw[i] = __builtin_amdgcn_ds_bpermute(fetch_from, raw[i]);
    vf[t] = *reinterpret_cast<s16x4*>(&raw);
  }
}

// ------------------------------------------------------------------ decode
// Split s of a token covers keys [s * 64 TPW, (s + 1) * 64 TPW); wavefront w of its
// workgroup takes the 16-key tiles w, w + 4, ... of the split, all loaded before the
// first is used.  Each workgroup leaves its partial result (unnormalised sums, running
// maximum and sum of weights per head) in `part_*`; a second kernel adds the partials
// in split order.  (Merging in the last workgroup to finish, found by a ticket
// counter, was tried: the device-wide fences it needs write back and invalidate L2
// for every workgroup and cost more than the second launch.)
//   part_acc[((token * nkv + kvh) * max_splits + split) * g + head in group][HD]
//   part_ml [ ... same index ... ][2] = (maximum in log2 units, sum)
template <int HD, int TPW>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    float* __restrict__ part_acc, float* __restrict__ part_ml, int max_splits,
    const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ dec_tok,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_tables,
    int max_blocks, int bs, int nh, int nkv, float scale_log2, int window) {
  constexpr int SPLIT = 64 * TPW;
  const int split = blockIdx.x, kvh = blockIdx.y;
  const int tok = dec_tok[blockIdx.z];
  const int pos[1] = {positions[tok]};
  const int start[1] = {(window > 0 && pos[0] - window + 1 > 0) ? pos[0] - window + 1 : 0};
  const int s_first = start[0] / SPLIT, s_last = pos[0] / SPLIT;
  if (split < s_first || split > s_last) return;
  const int lo = max(split * SPLIT, start[0] / 16 * 16);
  const int hi = min((split + 1) * SPLIT, pos[0] + 1);  // keys [lo, hi), not empty
  const int* table = block_tables + (int64_t)tok_seq[tok] * max_blocks;
  const int g = nh / nkv;
  const int lane = threadIdx.x % PAE_WAVE, wave = threadIdx.x / PAE_WAVE;
  const int col = lane % 16, g4 = lane / 16;

  bf16x8 qf[1][HD / 32];
  {
    const bf16_t* qrow = q + (int64_t)tok * q_stride + (int64_t)(kvh * g + (col < g ? col : 0)) * HD;
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) {
      qf[0][j] = *reinterpret_cast<const bf16x8*>(qrow + 32 * j + 8 * g4);
      if (col >= g)
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[0][j][e] = (__bf16)0.f;
    }
  }
  AttnState<HD, 1> st;
  st.m[0] = NEG_BIG;
  st.l[0] = 0.f;
#pragma unroll
  for (int t = 0; t < HD / 16; ++t) st.acc[0][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int page_elems = bs * HD;
  const int tile_lo = lo / 16, tile_hi = (hi + 15) / 16;
  bf16x8 kf[TPW][HD / 32];
  s16x4 vf[TPW][HD / 16];
#pragma unroll
  for (int j = 0; j < TPW; ++j) {  // a tile past the end is loaded from the first tile's place and not used
    const int tile = tile_lo + wave + 4 * j;
    const int key0 = (tile < tile_hi ? tile : tile_lo) * 16;
    const int64_t base = ((int64_t)table[key0 / bs] * nkv + kvh) * page_elems;
    load_kv_tile<HD>(kf[j], vf[j], k_cache + base + (int64_t)(key0 % bs) * HD, v_cache + base + key0 % bs, bs);
  }
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int tile = tile_lo + wave + 4 * j;
    kv_to_mfma_order<HD>(kf[j], vf[j]);  // in every lane of the wavefront, used or not
    if (tile < tile_hi) attn_tile<HD, 1>(st, kf[j], vf[j], qf, tile * 16, pos, start, scale_log2);
  }

  // wavefronts 1..3 hand their state to wavefront 0 through LDS; every lane of a wavefront
  // holds the same (column, features) as the same lane of wavefront 0
  extern __shared__ float s_buf[];  // [3][HD / 4 + 2][64]
  constexpr int ROWS = HD / 4 + 2;
  if (wave > 0) {
    float* mine = s_buf + (wave - 1) * ROWS * PAE_WAVE;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[(4 * t + i) * PAE_WAVE + lane] = st.acc[0][t][i];
    mine[(HD / 4) * PAE_WAVE + lane] = st.m[0];
    mine[(HD / 4 + 1) * PAE_WAVE + lane] = st.l[0];
  }
  __syncthreads();
  const int64_t group_slot = ((int64_t)blockIdx.z * nkv + kvh) * max_splits;
  if (wave == 0) {
#pragma unroll
    for (int w = 0; w < 3; ++w) {
      const float* theirs = s_buf + w * ROWS * PAE_WAVE;
      const float mw = theirs[(HD / 4) * PAE_WAVE + lane];
      const float m_new = fmaxf(st.m[0], mw);
      const float f0 = exp2f(st.m[0] - m_new), fw = exp2f(mw - m_new);
#pragma unroll
      for (int t = 0; t < HD / 16; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) st.acc[0][t][i] = st.acc[0][t][i] * f0 + theirs[(4 * t + i) * PAE_WAVE + lane] * fw;
      st.l[0] = st.l[0] * f0 + theirs[(HD / 4 + 1) * PAE_WAVE + lane] * fw;
      st.m[0] = m_new;
    }
    float l = st.l[0];
    l += __shfl_xor(l, 16, PAE_WAVE);
    l += __shfl_xor(l, 32, PAE_WAVE);
    if (col < g) {
      const int64_t slot = (group_slot + split) * g + col;
#pragma unroll
      for (int t = 0; t < HD / 16; ++t)
        *reinterpret_cast<f32x4*>(part_acc + slot * HD + 16 * t + 4 * g4) = st.acc[0][t];
      if (g4 == 0) {
        part_ml[slot * 2] = st.m[0];
        part_ml[slot * 2 + 1] = l;
      }
    }
  }
}

// Adds a token's partials in split order and writes the output: one workgroup per
// (token, kv head), one thread per (head of the group, four features), launched after
// the kernel above.  Kept small: it runs for microseconds.
template <int HD, int TPW>
__global__ void attn_decode_merge_kernel(bf16_t* __restrict__ out, int64_t out_stride,
                                         const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                                         int max_splits, const int* __restrict__ dec_tok,
                                         const int* __restrict__ positions, int nh, int nkv, int window) {
  constexpr int SPLIT = 64 * TPW;
  const int kvh = blockIdx.x;
  const int tok = dec_tok[blockIdx.y];
  const int pos = positions[tok];
  const int start = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int s_first = start / SPLIT, nsplits = pos / SPLIT - s_first + 1;
  const int g = nh / nkv;
  const int item = threadIdx.x;  // (head in group, chunk of four features)
  if (item >= g * (HD / 4)) return;
  const int c = item / (HD / 4), d = (item % (HD / 4)) * 4;
  const int64_t slot0 = (((int64_t)blockIdx.y * nkv + kvh) * max_splits + s_first) * g + c;
  float m = NEG_BIG, l = 0.f;
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int sp = 0; sp < nsplits; ++sp) {  // consecutive splits are g slots apart
    const int64_t slot = slot0 + (int64_t)sp * g;
    const float ms = part_ml[slot * 2], ls = part_ml[slot * 2 + 1];
    const f32x4 v = *reinterpret_cast<const f32x4*>(part_acc + slot * HD + d);
    const float m_new = fmaxf(m, ms);
    const float f_old = exp2f(m - m_new), f = exp2f(ms - m_new);
    a = a * f_old + v * f;
    l = l * f_old + ls * f;
    m = m_new;
  }
  const float inv = 1.0f / l;
  s16x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = bf16_bits(a[i] * inv);
  *reinterpret_cast<s16x4*>(out + (int64_t)tok * out_stride + (int64_t)(kvh * g + c) * HD + d) = w;
}

// ------------------------------------------------------------------ prefill
// tiles[t] = (row of the sequence in the tables, first flat token, number of tokens <= 32);
// the tokens of a tile are consecutive in the step and in position.
#define PREFILL_CT 2
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ tiles,
    int num_tiles, const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks,
    int bs, int nh, int nkv, float scale_log2, int window) {
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  const int tile_id = blockIdx.x * 4 + wave;
  if (tile_id >= num_tiles) return;
  const int head = blockIdx.y;
  const int kvh = head / (nh / nkv);
  const int seq_row = tiles[tile_id * 3], tok0 = tiles[tile_id * 3 + 1], ntok = tiles[tile_id * 3 + 2];
  const int* table = block_tables + (int64_t)seq_row * max_blocks;
  const int col = lane % 16, g4 = lane / 16;
  const int pos0 = positions[tok0];

  int pos[PREFILL_CT], start[PREFILL_CT];
  bf16x8 qf[PREFILL_CT][HD / 32];
  int lo = pos0, hi = pos0;  // keys any column needs: [lo, hi]
#pragma unroll
  for (int ct = 0; ct < PREFILL_CT; ++ct) {
    const int c = ct * 16 + col;
    const bool live = c < ntok;
    pos[ct] = live ? pos0 + c : -1;  // a dead column sees no key
    start[ct] = (live && window > 0 && pos[ct] - window + 1 > 0) ? pos[ct] - window + 1 : 0;
    const bf16_t* qrow = q + (int64_t)(tok0 + (live ? c : 0)) * q_stride + (int64_t)head * HD;
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) qf[ct][j] = *reinterpret_cast<const bf16x8*>(qrow + 32 * j + 8 * g4);
  }
  hi = pos0 + ntok - 1;
  lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;

  AttnState<HD, PREFILL_CT> st;
#pragma unroll
  for (int ct = 0; ct < PREFILL_CT; ++ct) {
    st.m[ct] = NEG_BIG;
    st.l[ct] = 0.f;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) st.acc[ct][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const int page_elems = bs * HD;
  bf16x8 kf[HD / 32];
  s16x4 vf[HD / 16];
  for (int key0 = lo / 16 * 16; key0 <= hi; key0 += 16) {
    const int blk = table[key0 / bs];
    const int64_t base = ((int64_t)blk * nkv + kvh) * page_elems;
    load_kv_tile<HD>(kf, vf, k_cache + base + (int64_t)(key0 % bs) * HD, v_cache + base + key0 % bs, bs);
    kv_to_mfma_order<HD>(kf, vf);
    attn_tile<HD, PREFILL_CT>(st, kf, vf, qf, key0, pos, start, scale_log2);
  }
#pragma unroll
  for (int ct = 0; ct < PREFILL_CT; ++ct) {
    float l = st.l[ct];
    l += __shfl_xor(l, 16, PAE_WAVE);
    l += __shfl_xor(l, 32, PAE_WAVE);
    const int c = ct * 16 + col;
    if (c >= ntok) continue;
    const float inv = 1.0f / l;
    bf16_t* o = out + (int64_t)(tok0 + c) * out_stride + (int64_t)head * HD;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) {
      s16x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = bf16_bits(st.acc[ct][t][i] * inv);
      *reinterpret_cast<s16x4*>(o + 16 * t + 4 * g4) = w;
    }
  }
}

// ------------------------------------------------------------------ entry points
#define FOR_HEAD_DIM(hd, CALL)                                       \
  switch (hd) {                                                      \
    case 32: { CALL(32); break; }                                    \
    case 64: { CALL(64); break; }                                    \
    case 96: { CALL(96); break; }                                    \
    case 128: { CALL(128); break; }                                  \
    case 160: { CALL(160); break; }                                  \
    case 192: { CALL(192); break; }                                  \
    case 224: { CALL(224); break; }                                  \
    case 256: { CALL(256); break; }                                  \
    default: return pae_fail("matrix-core attention takes head_dim in multiples of 32 up to 256, got %d", hd); \
  }

static int check_common(const char* what, int nh, int nkv, int hd, int bs, int max_blocks, int window) {
  PAE_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: %d query heads over %d key/value heads", what, nh, nkv);
  PAE_REQUIRE(nh / nkv <= 16, "%s: more than 16 query heads per key/value head (%d)", what, nh / nkv);
  PAE_REQUIRE(bs >= 16 && bs % 16 == 0, "%s: page size %d is not a multiple of 16", what, bs);
  PAE_REQUIRE(max_blocks > 0 && window >= 0, "%s: bad table width %d or window %d", what, max_blocks, window);
  PAE_REQUIRE(hd % 32 == 0 && hd >= 32 && hd <= 256, "%s: head_dim %d is not a multiple of 32 up to 256", what, hd);
  return 0;
}

// Keys per split of the decode kernel (fixed, so a token's result does not depend on the batch).
#define DECODE_TPW 2
extern "C" int pae_attn_decode_split() { return 64 * DECODE_TPW; }

// Workspace: part_acc holds num_dec * nh * max_splits * hd floats, part_ml num_dec * nh * max_splits * 2,
// max_splits = ceil(max_blocks * bs / pae_attn_decode_split()).
extern "C" int pae_attn_decode_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                    const void* k_cache, const void* v_cache, const int* dec_tok, int num_dec,
                                    const int* positions, const int* tok_seq, const int* block_tables,
                                    int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window,
                                    void* part_acc, void* part_ml, hipStream_t stream) {
  if (int rc = check_common("attn_decode", nh, nkv, hd, bs, max_blocks, window)) return rc;
  PAE_REQUIRE(num_dec <= 65535 && nkv <= 65535, "attn_decode: grid too large");
  if (num_dec <= 0) return 0;
  const int split_len = 64 * DECODE_TPW;
  const int max_splits = (int)(((int64_t)max_blocks * bs + split_len - 1) / split_len);
  const float scale_log2 = scale * LOG2E;
  dim3 grid(max_splits, nkv, num_dec), merge_grid(nkv, num_dec);
#define CALL(HD)                                                                                            \
  attn_decode_kernel<HD, DECODE_TPW><<<grid, 256, (size_t)3 * (HD / 4 + 2) * PAE_WAVE * sizeof(float), stream>>>( \
      (float*)part_acc, (float*)part_ml, max_splits, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,     \
      (const bf16_t*)v_cache, dec_tok, positions, tok_seq, block_tables, max_blocks, bs, nh, nkv, scale_log2, \
      window);                                                                                               \
  attn_decode_merge_kernel<HD, DECODE_TPW><<<merge_grid, (nh / nkv * (HD / 4) + 63) / 64 * 64, 0, stream>>>( \
      (bf16_t*)out, out_stride, (const float*)part_acc, (const float*)part_ml, max_splits, dec_tok, positions, \
      nh, nkv, window)
  FOR_HEAD_DIM(hd, CALL)
#undef CALL
  return pae_check_launch("attn_decode");
}

extern "C" int pae_attn_prefill_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                     const void* k_cache, const void* v_cache, const int* tiles, int num_tiles,
                                     const int* positions, const int* block_tables, int max_blocks, int bs,
                                     int nh, int nkv, int hd, float scale, int window, hipStream_t stream) {
  if (int rc = check_common("attn_prefill", nh, nkv, hd, bs, max_blocks, window)) return rc;
  PAE_REQUIRE(nh <= 65535, "attn_prefill: grid too large");
  if (num_tiles <= 0) return 0;
  const float scale_log2 = scale * LOG2E;
  dim3 grid((num_tiles + 3) / 4, nh);
#define CALL(HD)                                                                                          \
  attn_prefill_kernel<HD><<<grid, 256, 0, stream>>>((bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, \
                                                    (const bf16_t*)k_cache, (const bf16_t*)v_cache, tiles, \
                                                    num_tiles, positions, block_tables, max_blocks, bs, nh, \
                                                    nkv, scale_log2, window)
  FOR_HEAD_DIM(hd, CALL)
#undef CALL
  return pae_check_launch("attn_prefill");
}

// ------------------------------------------------------------------ prefill, long runs
// One workgroup per (up to 128 consecutive tokens of a sequence, query head); each of
// its four wavefronts owns 32 of the tokens.  Keys and values of BN keys at a time are
// staged in LDS by the whole workgroup (the next tile is fetched into registers while
// the current one is used) and every wavefront multiplies them with its own queries:
//   S^T[32 keys x 32 tokens] = K * Q^T             (MFMA 32x32x16, k = hd)
//   O^T[32 features x 32 tokens] += V^T * P^T      (MFMA 32x32x16, k = 16 keys)
// The accumulator of S^T holds, per lane (token = lane % 32, half = lane / 32), keys
// 8 j + 4 half + i of each 32-key block; two such groups of four are the 8 k-slots of a
// lane in the second product, whose A operand reads the values of exactly those keys.
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <int HD, int BN>
__global__ __launch_bounds__(256, HD <= 128 ? 2 : 1) void attn_prefill_lds_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks, int bs, int nh,
    int nkv, float scale_log2, int window) {
  constexpr int KS = HD + 8;   // row stride of the key tile in LDS (elements), padded against bank conflicts
  constexpr int VS = BN + 8;   // row stride of the transposed value tile
  constexpr int PAGES = BN / 16;
  constexpr int KCH = (16 * HD / 8 + 255) / 256;  // 16-byte chunks per thread and page
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[BN * KS];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[HD * VS];

  const int tid = threadIdx.x, wave = tid / PAE_WAVE, lane = tid % PAE_WAVE;
  const int col = lane % 32, half = lane / 32;
  const int head = blockIdx.y, kvh = head / (nh / nkv);
  const int seq_row = tiles[blockIdx.x * 3], tok0 = tiles[blockIdx.x * 3 + 1], ntok = tiles[blockIdx.x * 3 + 2];
  const int* table = block_tables + (int64_t)seq_row * max_blocks;
  const int pos0 = positions[tok0];
  const int c = wave * 32 + col;          // this lane's token within the tile
  const bool live = c < ntok;
  const int pos = live ? pos0 + c : -1;   // a dead column sees no key
  const int start = (live && window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int wave_hi = min(pos0 + wave * 32 + 31, pos0 + ntok - 1);  // last position of this wavefront
  const bool wave_live = wave * 32 < ntok;
  const bool wave_full = wave * 32 + 32 <= ntok;  // no dead column in this wavefront
  const int wave_lo = pos0 + wave * 32;            // its first position, and the window start of its last
  const int wave_start = (window > 0 && wave_hi - window + 1 > 0) ? wave_hi - window + 1 : 0;
  const int lo = (window > 0 && pos0 - window + 1 > 0) ? (pos0 - window + 1) / BN * BN : 0;
  const int hi = pos0 + ntok - 1;

  // queries: B operand, lane holds token `col`, features 16 ks + 8 half .. + 7
  bf16x8 qf[HD / 16];
  {
    const bf16_t* qrow = q + (int64_t)(tok0 + (live ? c : 0)) * q_stride + (int64_t)head * HD;
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + 16 * ks + 8 * half);
  }
  f32x16 acc[HD / 32];
#pragma unroll
  for (int t = 0; t < HD / 32; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
  float m = NEG_BIG, l = 0.f;

  const int page_elems = bs * HD;
  // staging registers: per page, this thread's 16-byte chunks of the key page and of the value page
  bf16x8 kreg[PAGES][KCH], vreg[PAGES][KCH];
  auto fetch = [&](int key0) {
#pragma unroll
    for (int p = 0; p < PAGES; ++p) {
      const int key = key0 + 16 * p;
      const int kc = key <= hi ? key : key0;  // pages past the end repeat the first one (never used)
      // a page the window has passed was given back (its entry is -1): every key of it is masked, read page 0
      const int64_t base = ((int64_t)max(table[kc / bs], 0) * nkv + kvh) * page_elems;
      const bf16_t* kp = k_cache + base + (int64_t)(kc % bs) * HD;  // [16 keys][HD], contiguous
      const bf16_t* vp = v_cache + base + kc % bs;                  // [HD][bs]: 16 keys of each feature
#pragma unroll
      for (int ch = 0; ch < KCH; ++ch) {
        const int idx = tid + 256 * ch;  // chunk index within the page: 16 * HD / 8 chunks
        if (idx < 16 * HD / 8) {
          kreg[p][ch] = *reinterpret_cast<const bf16x8*>(kp + idx * 8);
          const int d = idx / 2, part = idx % 2;  // feature, which 8 of the 16 keys
          vreg[p][ch] = *reinterpret_cast<const bf16x8*>(vp + (int64_t)d * bs + 8 * part);
        }
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int p = 0; p < PAGES; ++p)
#pragma unroll
      for (int ch = 0; ch < KCH; ++ch) {
        const int idx = tid + 256 * ch;
        if (idx < 16 * HD / 8) {
          const int key = idx / (HD / 8), kchunk = idx % (HD / 8);
          *reinterpret_cast<bf16x8*>(k_lds + (16 * p + key) * KS + 8 * kchunk) = kreg[p][ch];
          const int d = idx / 2, part = idx % 2;
          *reinterpret_cast<bf16x8*>(v_lds + d * VS + 16 * p + 8 * part) = vreg[p][ch];
        }
      }
  };

  fetch(lo);
  for (int key0 = lo; key0 <= hi; key0 += BN) {
    __syncthreads();  // the previous tile has been read by every wavefront
    stage();
    __syncthreads();
    if (key0 + BN <= hi) fetch(key0 + BN);
    if (!wave_live || key0 > wave_hi) continue;  // nothing for this wavefront in the tile (causal)
    // scores of the whole tile first, then one softmax update and one rescale for it
    f32x16 s[BN / 32];
#pragma unroll
    for (int kb = 0; kb < BN / 32; ++kb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
      bf16x8 kf[HD / 16];  // all key fragments of the block are read before the first product uses one
#pragma unroll
      for (int ks = 0; ks < HD / 16; ++ks)
        kf[ks] = *reinterpret_cast<const bf16x8*>(k_lds + (32 * kb + col) * KS + 16 * ks + 8 * half);
#pragma unroll
      for (int ks = 0; ks < HD / 16; ++ks) s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], s[kb], 0, 0, 0);
    }
    // a tile that every token of this wavefront sees whole needs no mask
    const bool whole = wave_full && key0 + BN - 1 <= wave_lo && key0 >= wave_start;
    float mx = NEG_BIG;
    if (whole) {
#pragma unroll
      for (int kb = 0; kb < BN / 32; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          s[kb][v] *= scale_log2;
          mx = fmaxf(mx, s[kb][v]);
        }
    } else {
#pragma unroll
      for (int kb = 0; kb < BN / 32; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = key0 + 32 * kb + 8 * (v / 4) + 4 * half + v % 4;
          s[kb][v] = (key <= pos && key >= start) ? s[kb][v] * scale_log2 : -INFINITY;
          mx = fmaxf(mx, s[kb][v]);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, PAE_WAVE));
    const float m_new = fmaxf(m, mx);
    const float alpha = exp2f(m - m_new);
    m = m_new;
    float psum = 0.f;
    bf16x8 pb[BN / 32][2];
#pragma unroll
    for (int kb = 0; kb < BN / 32; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float p = exp2f(s[kb][v] - m_new);
        psum += p;
        pb[kb][v / 8][v % 8] = (__bf16)p;
      }
    l = l * alpha + psum;
#pragma unroll
    for (int t = 0; t < HD / 32; ++t) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][v] *= alpha;
      // value fragments: keys 16 st + 4 half + (0..3) and 16 st + 8 + 4 half + (0..3) of block kb, feature 32 t + col
      bf16x8 vf[BN / 32][2];
#pragma unroll
      for (int kb = 0; kb < BN / 32; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const bf16_t* vrow = v_lds + (32 * t + col) * VS + 32 * kb + 16 * st + 4 * half;
          s16x4* dst = reinterpret_cast<s16x4*>(&vf[kb][st]);
          dst[0] = *reinterpret_cast<const s16x4*>(vrow);
          dst[1] = *reinterpret_cast<const s16x4*>(vrow + 8);
        }
#pragma unroll
      for (int kb = 0; kb < BN / 32; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kb][st], pb[kb][st], acc[t], 0, 0, 0);
    }
  }
  l += __shfl_xor(l, 32, PAE_WAVE);
  if (!live) return;
  const float inv = 1.0f / l;
  bf16_t* o = out + (int64_t)(tok0 + c) * out_stride + (int64_t)head * HD;
#pragma unroll
  for (int t = 0; t < HD / 32; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // registers 4 j .. 4 j + 3 are features 32 t + 8 j + 4 half + (0..3)
      s16x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = bf16_bits(acc[t][4 * j + i] * inv);
      *reinterpret_cast<s16x4*>(o + 32 * t + 8 * j + 4 * half) = w;
    }
}

// tiles[t] = (table row of the sequence, first flat token, number of tokens <= 128)
extern "C" int pae_attn_prefill_long_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                          const void* k_cache, const void* v_cache, const int* tiles,
                                          int num_tiles, const int* positions, const int* block_tables,
                                          int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window,
                                          hipStream_t stream) {
  if (int rc = check_common("attn_prefill_long", nh, nkv, hd, bs, max_blocks, window)) return rc;
  PAE_REQUIRE(nh <= 65535, "attn_prefill_long: grid too large");
  if (num_tiles <= 0) return 0;
  const float scale_log2 = scale * LOG2E;
  dim3 grid(num_tiles, nh);
#define CALL(HD)                                                                                            \
  attn_prefill_lds_kernel<HD, (HD <= 128 ? 64 : 32)><<<grid, 256, 0, stream>>>(                             \
      (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, \
      tiles, positions, block_tables, max_blocks, bs, nh, nkv, scale_log2, window)
  FOR_HEAD_DIM(hd, CALL)
#undef CALL
  return pae_check_launch("attn_prefill_long");
}
