// Causal attention over the paged cache on the matrix cores (bfloat16 in,
// float32 scores, softmax and accumulation).
//
// Both kernels work on transposed tiles so that the softmax output can feed the
// second product without leaving registers:
//   S^T[16 keys x 16 columns] = K[16 keys x hd] * Q^T        (MFMA 16x16x32, k = hd)
//   O^T[hd x 16 columns]     += V^T[hd x keys] * P^T          (k = 16 keys in the decode kernel,
//                                                             32 keys of two pages in the prefill kernel)
// The accumulator layout of S^T (lane = column, registers = 4 consecutive keys) is
// exactly the B-operand layout of the second product.  A "column" is one (token,
// query head); the 16 keys of a tile are one cache page (or a 16-key slice of a
// larger page).  Keys live as [block][kv head][page][hd], values transposed as
// [block][kv head][hd][page], so both A operands are contiguous in memory; they are loaded
// with a quad of lanes on contiguous bytes and moved to the instruction's lane order by
// cross-lane permutes (see `load_kv_tile`).
//
// decode:  one workgroup per (sequence with a single new token, kv head, split of
//          the keys); the columns are the query heads that share the kv head, so a
//          page is read once for all of them.  Four wavefronts take pages in turn
//          and merge in LDS; a second small kernel merges the splits.  Splits
//          start at multiples of the split length from position 0.
// prefill: one workgroup per (up to 64 consecutive tokens of a sequence, query head), whose
//          wavefronts share out the keys (see there).
//
// Masking is the reference's rule (engine/attention.py:474-487: key j visible iff
// j <= position of the query) plus an optional window.  A column's result depends
// only on its own position: fully masked pages add exact zeros.
#include "common.h"
#include "api.h"
#include "attention_device.h"

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
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int4* __restrict__ dec_work,
    const int* __restrict__ block_tables, int max_blocks, int bs, int nh, int nkv, float scale_log2, int window) {
  constexpr int SPLIT = 64 * TPW;
  const int split = blockIdx.x, kvh = blockIdx.y;
  // one load brings the token's row, its position and its table row: a chain of three dependent
  // loads (token, then position and sequence, then pages) would cost a trip to memory each
  const int4 work = dec_work[blockIdx.z];
  // In a step of single tokens only, token i's sequence is row i of the tables: this wavefront's table
  // entries are asked for from that row together with the work item, not after it, and used if the
  // item then names that row (one trip to memory fewer before the keys can be asked for).
  const int lane = threadIdx.x % PAE_WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE);
  int guessed[TPW];
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int page = (split * (SPLIT / 16) + wave + 4 * j) * 16 / bs;
    guessed[j] = block_tables[(int64_t)blockIdx.z * max_blocks + (page < max_blocks ? page : max_blocks - 1)];
  }
  const int tok = work.x;
  const int pos[1] = {work.y};
  const int start[1] = {(window > 0 && pos[0] - window + 1 > 0) ? pos[0] - window + 1 : 0};
  const int s_first = start[0] / SPLIT, s_last = pos[0] / SPLIT;
  if (split < s_first || split > s_last) return;
  const int lo = max(split * SPLIT, start[0] / 16 * 16);
  const int hi = min((split + 1) * SPLIT, pos[0] + 1);  // keys [lo, hi), not empty
  const int* table = block_tables + (int64_t)work.z * max_blocks;
  const int g = nh / nkv;
  // (the wavefront's number is a scalar, so that its pages' table entries come by scalar loads)
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
    const bool as_guessed = work.z == (int)blockIdx.z && key0 / 16 == split * (SPLIT / 16) + wave + 4 * j;
    const int64_t base = ((int64_t)(as_guessed ? guessed[j] : table[key0 / bs]) * nkv + kvh) * page_elems;
    load_kv_tile<HD>(kf[j], vf[j], k_cache + base + (int64_t)(key0 % bs) * HD, v_cache + base + key0 % bs, bs);
  }
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int tile = tile_lo + wave + 4 * j;
    keys_to_mfma_order<HD>(kf[j]);  // in every lane of the wavefront, used or not
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
                                         int max_splits, const int4* __restrict__ dec_work, int nh, int nkv,
                                         int window) {
  // blockDim = (items rounded up to wavefronts, G): the splits are dealt out to G groups of threads,
  // whose loads are all in flight together; group 0 then adds the groups' sums in group order.
  extern __shared__ float s_merge[];  // [G - 1][items][6]: four sums, maximum, sum of weights
  constexpr int SPLIT = 64 * TPW;
  const int kvh = blockIdx.x;
  const int4 work = dec_work[blockIdx.y];
  const int tok = work.x, pos = work.y;
  const int start = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int s_first = start / SPLIT, nsplits = pos / SPLIT - s_first + 1;
  const int g = nh / nkv, items = g * (HD / 4);
  const int item = threadIdx.x, group = threadIdx.y, groups = blockDim.y;  // item: (head in group, four features)
  const bool live = item < items;
  const int c = live ? item / (HD / 4) : 0, d = (item % (HD / 4)) * 4;
  const int64_t slot0 = (((int64_t)blockIdx.y * nkv + kvh) * max_splits + s_first) * g + c;
  float m = NEG_BIG, l = 0.f;
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
  if (live) {
#pragma unroll 8
    for (int sp = group; sp < nsplits; sp += groups) {  // consecutive splits are g slots apart
      const int64_t slot = slot0 + (int64_t)sp * g;
      const float ms = part_ml[slot * 2], ls = part_ml[slot * 2 + 1];
      const f32x4 v = *reinterpret_cast<const f32x4*>(part_acc + slot * HD + d);
      const float m_new = fmaxf(m, ms);
      const float f_old = exp2f(m - m_new), f = exp2f(ms - m_new);
      a = a * f_old + v * f;
      l = l * f_old + ls * f;
      m = m_new;
    }
    if (group > 0) {
      float* dst = s_merge + ((int64_t)(group - 1) * items + item) * 6;
      dst[0] = a[0]; dst[1] = a[1]; dst[2] = a[2]; dst[3] = a[3]; dst[4] = m; dst[5] = l;
    }
  }
  __syncthreads();
  if (!live || group > 0) return;
  for (int other = 1; other < groups; ++other) {
    const float* src = s_merge + ((int64_t)(other - 1) * items + item) * 6;
    const float ms = src[4], ls = src[5];
    const float m_new = fmaxf(m, ms);
    const float f_old = exp2f(m - m_new), f = exp2f(ms - m_new);
    a = a * f_old + (f32x4){src[0], src[1], src[2], src[3]} * f;
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
// One workgroup per (run of up to 16 CT consecutive tokens of a sequence, query head).  All four
// wavefronts hold the run's queries (B operands of the first product) and take the keys in
// turn, 32 at a time: wavefront w takes keys [lo + 32 (w + 4 i), + 32).  Every wavefront reads
// its own keys and values straight from the cache into registers, so the loop has no barrier.
// Keys and values have one register set each, refilled as soon as the product that read it has
// been issued: the next keys arrive during the softmax and the second product, the next values
// during the following first product.  At the end the four partial results (reference, sum,
// unnormalised output) are merged through LDS, column tile ct by wavefront ct.
//
// The softmax keeps, per column, a reference value that is at most RESCALE_STEP (in units of log2)
// below the largest score seen: weights are exp2(score - reference), at most 2^RESCALE_STEP, and the
// sums so far are rescaled only when a score passes reference + RESCALE_STEP (then the reference
// becomes the column's maximum).  Any reference gives the same quotient sum(w v) / sum(w); a stale
// one saves rescaling the whole output tile for every 32 keys, which costs more than the products.
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
#define RESCALE_STEP 8.0f

// A register loaded in the order (row = lane / 4, group = lane % 4), in which a quad of lanes reads
// contiguous bytes, moved to the matrix instruction's order (row = lane % 16, group = lane / 16).
__device__ __forceinline__ bf16x8 quad_to_mfma_order(bf16x8 x, int fetch_from) {
  i32x4 raw = *reinterpret_cast<i32x4*>(&x);
#pragma unroll
  for (int i = 0; i < 4; ++i) raw[i] = __builtin_amdgcn_ds_bpermute(fetch_from, raw[i]);
  return *reinterpret_cast<bf16x8*>(&raw);
}

// tiles[t] = (table row of the sequence, first flat token, number of tokens <= 64); blockIdx.z picks
// the part of 16 CT tokens of the run that this workgroup takes.
// BS: the page size if it is 16 (the value rows' offsets are then constants), or 0 for any other.
template <int HD, int CT, int BS>
__global__ __launch_bounds__(256, 1) void attn_prefill_split_kernel(
    bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks, int bs, int nh,
    int nkv, float scale_log2, int window) {
  constexpr int UNIT = 32, TOK = 16 * CT;
  if (BS) bs = BS;
  __shared__ float s_acc[3][HD / 16][4][PAE_WAVE];
  __shared__ float s_ml[3][2][PAE_WAVE];

  // the wavefront's number as a scalar: what is computed from it (the keys it takes, their pages'
  // table entries) then lives in scalar registers and is loaded by scalar loads, which the vector
  // loads' in-order counter does not wait for (as a vector load, every table lookup waited for all
  // keys and values in flight)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE), lane = threadIdx.x % PAE_WAVE;
  const int col = lane % 16, g4 = lane / 16;
  const int head = blockIdx.x, kvh = head / (nh / nkv);
  const int seq_row = tiles[blockIdx.y * 3];
  const int tok0 = tiles[blockIdx.y * 3 + 1] + blockIdx.z * TOK;
  const int ntok = min(TOK, tiles[blockIdx.y * 3 + 2] - (int)blockIdx.z * TOK);
  if (ntok <= 0) return;  // the whole workgroup
  const int* table = block_tables + (int64_t)seq_row * max_blocks;
  const int pos0 = positions[tok0];

  int pos[CT], start[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + col;
    const bool live = c < ntok;
    pos[ct] = live ? pos0 + c : -1;  // a dead column sees no key
    start[ct] = (live && window > 0 && pos[ct] - window + 1 > 0) ? pos[ct] - window + 1 : 0;
  }
  bf16x8 qf[CT][HD / 32];  // B operands of the first product: column tile ct, features 32 j ..
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + col;
    const bf16_t* qrow = q + (int64_t)(tok0 + (c < ntok ? c : 0)) * q_stride + (int64_t)head * HD;
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) qf[ct][j] = *reinterpret_cast<const bf16x8*>(qrow + 32 * j + 8 * g4);
  }
  const int hi = pos0 + ntok - 1;                                                        // last key any token sees
  const int lo = (window > 0 && pos0 - window + 1 > 0) ? (pos0 - window + 1) / UNIT * UNIT : 0;  // first, rounded down
  const int last_start = (window > 0 && hi - window + 1 > 0) ? hi - window + 1 : 0;     // window start of the last token

  f32x4 acc[CT][HD / 16];  // O^T: rows hd = 16 t + 4 g4 + i, column = lane % 16
  float ref[CT], l[CT];    // the column's reference (log2 units) and this lane's share of its sum of weights
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    ref[ct] = NEG_BIG;
    l[ct] = 0.f;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) acc[ct][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // Keys are loaded in the order (row = lane / 4, group = lane % 4), in which a quad of lanes reads
  // 64 contiguous bytes of a key row, and moved to the instruction's order by a permute.  kf[p][j]:
  // keys of page p, features 32 j ..  Values are loaded in the instruction's own order, feature
  // 16 t + lane % 16, keys 4 (lane / 16) .. + 3 of both pages: a quad's four pieces then lie in one
  // 128-byte line (value rows are 2 * page size bytes apart), which the memory pipeline takes as
  // well as contiguous ones, and the permutes are saved (378 -> 353 us at 8,192 tokens; keys, whose
  // rows are 2 * head_dim bytes apart, gain nothing without theirs).  vf[t]'s 8 k slots per lane
  // are exactly the scores the lane holds after the first product.
  const int lrow = lane / 4, lgrp = lane % 4;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;
  const int page_elems = bs * HD;
  bf16x8 kf[2][HD / 32], vf[HD / 16];
  auto page_base = [&](int key0, int p) -> int64_t {
    const int key = key0 + 16 * p;
    const int kc = key <= hi ? key : key0;  // a tile past the end repeats the first one (all of it is masked)
    // a page the window has passed was given back (its entry is -1): all its keys are masked, read page 0
    return ((int64_t)max(table[kc / bs], 0) * nkv + kvh) * page_elems;
  };
  auto load_keys = [&](int key0) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int key = key0 + 16 * p, kc = key <= hi ? key : key0;
      const bf16_t* kp = k_cache + page_base(key0, p) + (int64_t)(kc % bs) * HD;
#pragma unroll
      for (int j = 0; j < HD / 32; ++j) kf[p][j] = *reinterpret_cast<const bf16x8*>(kp + lrow * HD + 32 * j + 8 * lgrp);
    }
  };
  auto load_values = [&](int key0) {
    const bf16_t* vp[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int key = key0 + 16 * p, kc = key <= hi ? key : key0;
      vp[p] = v_cache + page_base(key0, p) + kc % bs;
    }
#pragma unroll
    for (int t = 0; t < HD / 16; ++t)  // in the order of their use
#pragma unroll
      for (int p = 0; p < 2; ++p)
        reinterpret_cast<bf16x4*>(&vf[t])[p] = *reinterpret_cast<const bf16x4*>(vp[p] + (int64_t)(16 * t + col) * bs + 4 * g4);
  };

  int key0 = lo + UNIT * wave;  // the same in every lane of a wavefront: the branches on it are uniform
  if (key0 <= hi) {
    load_keys(key0);
    load_values(key0);
  }
  for (; key0 <= hi; key0 += 4 * UNIT) {
    const bool more = key0 + 4 * UNIT <= hi;
    // The queries stay in the accumulation registers, which the matrix instruction reads directly:
    // the other half of the register file is needed for the keys, values and scores in flight.
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int j = 0; j < HD / 32; ++j) asm volatile("" : "+a"(qf[ct][j]));
    // scores of the 32 keys for every column tile
    f32x4 s[CT][2];
    {
      bf16x8 ka[2][HD / 32];
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int j = 0; j < HD / 32; ++j) ka[p][j] = quad_to_mfma_order(kf[p][j], fetch_from);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          s[ct][p] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < HD / 32; ++j)
            s[ct][p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[p][j], qf[ct][j], s[ct][p], 0, 0, 0);
        }
    }
    if (more) load_keys(key0 + 4 * UNIT);  // into the registers the first product has just read
    if (!(key0 + UNIT - 1 <= pos0 && key0 >= last_start)) {  // some key is hidden from some token of the run
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = key0 + 16 * p + 4 * g4 + i;
            if (!(key <= pos[ct] && key >= start[ct])) s[ct][p][i] = -INFINITY;
          }
    }
    // does any score pass its column's reference by more than the step?  (each lane for its own scores)
    float mx[CT];
    bool passed = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      mx[ct] = fmaxf(fmaxf(fmaxf(s[ct][0][0], s[ct][0][1]), fmaxf(s[ct][0][2], s[ct][0][3])),
                     fmaxf(fmaxf(s[ct][1][0], s[ct][1][1]), fmaxf(s[ct][1][2], s[ct][1][3]))) * scale_log2;
      passed |= mx[ct] > ref[ct] + RESCALE_STEP;
    }
    if (__builtin_amdgcn_ballot_w64(passed) != 0) {  // the same in every lane; rare after the first units
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) asm volatile("" : "+a"(acc[ct][t]));  // moved from there only in here
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        float m = fmaxf(mx[ct], NEG_BIG);
        m = fmaxf(m, __shfl_xor(m, 16, PAE_WAVE));
        m = fmaxf(m, __shfl_xor(m, 32, PAE_WAVE));  // the column's maximum in this unit
        const float to = m > ref[ct] + RESCALE_STEP ? m : ref[ct];
        const float alpha = __builtin_amdgcn_exp2f(ref[ct] - to);
        ref[ct] = to;
        l[ct] *= alpha;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) acc[ct][t] *= alpha;
      }
    }
    // the sums are in the accumulation registers on both ways here (or the compiler moves the whole
    // output tile to ordinary registers and back in every pass for the sake of the rare branch)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int t = 0; t < HD / 16; ++t) asm volatile("" : "+a"(acc[ct][t]));
    // Column tile by column tile: the weights of one (exponentials, sum, rounding: vector ALU), then
    // its second product (matrix pipe), so that the next tile's arithmetic can run under this
    // tile's products.
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      float w[8];
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          w[4 * p + i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ct][p][i], scale_log2, -ref[ct]));
      l[ct] += ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
      bf16x8 pb;
      bf16x2* pairs = reinterpret_cast<bf16x2*>(&pb);
#pragma unroll
      for (int i = 0; i < 4; ++i) pairs[i] = __builtin_convertvector((f32x2){w[2 * i], w[2 * i + 1]}, bf16x2);
#pragma unroll
      for (int t = 0; t < HD / 16; ++t) acc[ct][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t], pb, acc[ct][t], 0, 0, 0);
    }
    // Order asked of the compiler's scheduler for the above: the first tile's arithmetic, then one
    // matrix instruction and two vector instructions in turn (left alone it puts all exponentials
    // first and all products last, and each pipe idles while the other runs).
    __builtin_amdgcn_sched_group_barrier(0x002, 20, 0);
#pragma unroll
    for (int i = 0; i < CT * (HD / 16); ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
    }
    if (more) load_values(key0 + 4 * UNIT);
  }

  // merge: column tile ct is summed by wavefront ct from its own state and the three others' in LDS
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float sum = l[ct];
    sum += __shfl_xor(sum, 16, PAE_WAVE);
    sum += __shfl_xor(sum, 32, PAE_WAVE);
    l[ct] = sum;
  }
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int merger = ct % 4;
    if (wave != merger) {
      const int slot = wave < merger ? wave : wave - 1;
#pragma unroll
      for (int t = 0; t < HD / 16; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_acc[slot][t][i][lane] = acc[ct][t][i];
      s_ml[slot][0][lane] = ref[ct];
      s_ml[slot][1][lane] = l[ct];
    }
    __syncthreads();
    if (wave == merger) {
      float m = ref[ct];
#pragma unroll
      for (int w = 0; w < 3; ++w) m = fmaxf(m, s_ml[w][0][lane]);
      const float own = exp2f(ref[ct] - m);
      float sum = l[ct] * own;
      float scale_w[3];
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        scale_w[w] = exp2f(s_ml[w][0][lane] - m);
        sum += s_ml[w][1][lane] * scale_w[w];
      }
      const int c = ct * 16 + col;
      if (c < ntok) {
        const float inv = 1.0f / sum;
        bf16_t* o = out + (int64_t)(tok0 + c) * out_stride + (int64_t)head * HD;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) {
          s16x4 w4;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float a = acc[ct][t][i] * own;
#pragma unroll
            for (int w = 0; w < 3; ++w) a += s_acc[w][t][i][lane] * scale_w[w];
            w4[i] = bf16_bits(a * inv);
          }
          *reinterpret_cast<s16x4*>(o + 16 * t + 4 * g4) = w4;
        }
      }
    }
    __syncthreads();
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

// dec_work[i] = (flat row of the token, its position, row of its sequence in block_tables, unused),
// 16 bytes each, 16-byte aligned.
// Workspace: part_acc holds num_dec * nh * max_splits * hd floats, part_ml num_dec * nh * max_splits * 2,
// max_splits = ceil(max_blocks * bs / pae_attn_decode_split()).
extern "C" int pae_attn_decode_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                    const void* k_cache, const void* v_cache, const int* dec_work, int num_dec,
                                    const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window,
                                    void* part_acc, void* part_ml, hipStream_t stream) {
  if (int rc = check_common("attn_decode", nh, nkv, hd, bs, max_blocks, window)) return rc;
  PAE_REQUIRE(num_dec <= 65535 && nkv <= 65535, "attn_decode: grid too large");
  if (num_dec <= 0) return 0;
  const int split_len = 64 * DECODE_TPW;
  const int max_splits = (int)(((int64_t)max_blocks * bs + split_len - 1) / split_len);
  const float scale_log2 = scale * LOG2E;
  dim3 grid(max_splits, nkv, num_dec), merge_grid(nkv, num_dec);
  // merge: one thread per (head of the group, four features) and group of splits; four groups as far as
  // 1,024 threads go, whatever the number of splits (a group without splits adds exact zeros), so that
  // the order of adding depends on the head geometry alone
  const int merge_items = nh / nkv * (hd / 4);
  const int merge_x = (merge_items + PAE_WAVE - 1) / PAE_WAVE * PAE_WAVE;
  int merge_groups = 1024 / merge_x < 4 ? 1024 / merge_x : 4;
  if (merge_groups < 1) merge_groups = 1;
  PAE_REQUIRE(merge_x <= 1024, "attn_decode: %d heads of %d features per key/value head exceed the merge's workgroup", nh / nkv, hd);
  const size_t merge_lds = (size_t)(merge_groups - 1) * merge_items * 6 * sizeof(float);
#define CALL(HD)                                                                                            \
  attn_decode_kernel<HD, DECODE_TPW><<<grid, 256, (size_t)3 * (HD / 4 + 2) * PAE_WAVE * sizeof(float), stream>>>( \
      (float*)part_acc, (float*)part_ml, max_splits, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,     \
      (const bf16_t*)v_cache, (const int4*)dec_work, block_tables, max_blocks, bs, nh, nkv, scale_log2, \
      window);                                                                                               \
  attn_decode_merge_kernel<HD, DECODE_TPW><<<merge_grid, dim3(merge_x, merge_groups), merge_lds, stream>>>( \
      (bf16_t*)out, out_stride, (const float*)part_acc, (const float*)part_ml, max_splits, (const int4*)dec_work, \
      nh, nkv, window)
  FOR_HEAD_DIM(hd, CALL)
#undef CALL
  return pae_check_launch("attn_decode");
}

// tiles[t] = (table row of the sequence, first flat token, number of tokens <= 64), heaviest runs
// first: workgroups start in the order of the grid, and the last to finish sets the time.
extern "C" int pae_attn_prefill_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                          const void* k_cache, const void* v_cache, const int* tiles,
                                          int num_tiles, const int* positions, const int* block_tables,
                                          int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window,
                                          hipStream_t stream) {
  if (int rc = check_common("attn_prefill", nh, nkv, hd, bs, max_blocks, window)) return rc;
  PAE_REQUIRE(num_tiles <= 65535, "attn_prefill: %d runs exceed the grid", num_tiles);
  if (num_tiles <= 0) return 0;
  const float scale_log2 = scale * LOG2E;
  // Four column tiles (64 tokens) per workgroup up to head_dim 128, two above (registers).  Two also up to
  // head_dim 128 while the 64-token workgroups would not fill the chip's compute units: twice the
  // workgroups, each with half the arithmetic per 32 keys (1.5B heads: 512 tokens 16.4 -> 12.1 us, 1,024
  // tokens 22.0 -> 19.3; from 2,048 tokens on, 384 workgroups, four tiles are ahead: 40.5 against 47.0 us).
  const bool halves = (int64_t)nh * num_tiles <= 256;
#define LAUNCH_CT(HD, CT, BS)                                                                                  \
  attn_prefill_split_kernel<HD, CT, BS><<<dim3(nh, num_tiles, 4 / CT), 256, 0, stream>>>(                      \
      (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,    \
      tiles, positions, block_tables, max_blocks, bs, nh, nkv, scale_log2, window)
#define LAUNCH(HD, BS)                  \
  if (HD > 128 || halves) {             \
    LAUNCH_CT(HD, 2, BS);               \
  } else {                              \
    LAUNCH_CT(HD, (HD <= 128 ? 4 : 2), BS); \
  }
#define CALL(HD)        \
  if (bs == 16) {       \
    LAUNCH(HD, 16);     \
  } else {              \
    LAUNCH(HD, 0);      \
  }
  FOR_HEAD_DIM(hd, CALL)
#undef CALL
#undef LAUNCH
#undef LAUNCH_CT
  return pae_check_launch("attn_prefill");
}
