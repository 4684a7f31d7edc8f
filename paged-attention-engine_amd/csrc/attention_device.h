// Device code shared by the matrix-core attention kernels (attention_mfma.hip) and the decode program
// (decode_program.hip): one 16-key tile of scores, softmax weights and the second product, and the
// loads of a tile's keys and values from the paged cache.
#pragma once
#include "common.h"

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

// Keys are loaded with the lane order (row = lane / 4, group = lane % 4), so that the four lanes of
// a quad read 64 contiguous bytes of a key row and the memory pipeline sees one access for them;
// `keys_to_mfma_order` then moves every register to the order the matrix instruction wants
// (row = lane % 16, group = lane / 16) with one cross-lane permute each.  Values are loaded in the
// instruction's order at once: a quad's four 8-byte pieces lie in rows 2 * page size bytes apart,
// one 128-byte line at page size 16, which costs the pipeline no more and saves the permutes.
template <int HD>
__device__ __forceinline__ void load_kv_tile(bf16x8 (&kf)[HD / 32], s16x4 (&vf)[HD / 16], const bf16_t* kp,
                                             const bf16_t* vp, int vstride) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int r = lane / 4, g = lane % 4;
#pragma unroll
  for (int j = 0; j < HD / 32; ++j) kf[j] = *reinterpret_cast<const bf16x8*>(kp + r * HD + 32 * j + 8 * g);
#pragma unroll
  for (int t = 0; t < HD / 16; ++t)
    vf[t] = *reinterpret_cast<const s16x4*>(vp + (int64_t)(16 * t + lane % 16) * vstride + 4 * (lane / 16));
}

template <int HD>
__device__ __forceinline__ void keys_to_mfma_order(bf16x8 (&kf)[HD / 32]) {
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  const int lane = threadIdx.x % PAE_WAVE;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;  // byte address of the source lane
#pragma unroll
  for (int j = 0; j < HD / 32; ++j) {
    i32x4 raw = *reinterpret_cast<i32x4*>(&kf[j]);
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = __builtin_amdgcn_ds_bpermute(fetch_from, raw[i]);
    kf[j] = *reinterpret_cast<bf16x8*>(&raw);
  }
}

