// Causal attention over the paged cache, one wavefront per (token, query head).
//
// This is the kernel every size goes through in float32 and the one bfloat16
// falls back to when the matrix-core kernels do not take a shape.  A step's
// tokens are flat: token t belongs to sequence tok_seq[t] and stands at
// positions[t]; its keys are the cache slots of positions start..pos of that
// sequence, start = max(0, pos - window + 1) (window 0: every earlier key).  The
// rule is the reference's mask (engine/attention.py:474-487: key j is visible iff
// j <= query position and j < kv length) plus the window, which it lacks.
// KV head j serves query heads j*g .. (j+1)*g-1 (engine/attention.py:72-74).
//
// Keys are walked in chunks of 64 aligned to multiples of 64 from position 0,
// lane = key within the chunk, with an online softmax in float32.  What a
// (token, head) computes therefore depends on nothing but its own position:
// not on how the step was cut, nor on what else is in the batch.
#include "common.h"
#include "api.h"

template <typename T, int MAXD>  // MAXD: output features per lane, head_dim <= 64 * MAXD
__global__ void paged_attention_generic_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ tok_seq, const int* __restrict__ block_tables, int max_blocks, int bs,
    int nh, int nkv, int hd, float scale, int window) {
  extern __shared__ float lds[];  // [hd] query, [64] probabilities
  float* q_lds = lds;
  float* p_lds = lds + hd;
  const int t = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = head / (nh / nkv);
  const int pos = positions[t];
  const int* table = block_tables + (int64_t)tok_seq[t] * max_blocks;
  const int start = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  const T* q_row = q + (int64_t)t * q_stride + (int64_t)head * hd;
  for (int d = lane; d < hd; d += PAE_WAVE) q_lds[d] = to_f32(q_row[d]);
  __syncthreads();

  float acc[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int base = (start / PAE_WAVE) * PAE_WAVE; base <= pos; base += PAE_WAVE) {
    const int key = base + lane;
    const bool valid = key >= start && key <= pos;
    int row = 0;  // this lane's key row in the pool, in units of head_dim elements
    float s = -INFINITY;
    if (valid) {
      const int blk = table[key / bs];
      row = (blk * nkv + kvh) * bs + key % bs;
      const T* kr = k_cache + (int64_t)row * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_lds[d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: every chunk holds a valid key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);        // 0 on the first chunk (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_lds[lane] = p;
    __syncthreads();
    const int first = (start > base ? start - base : 0);
    const int last = (pos - base < PAE_WAVE - 1 ? pos - base : PAE_WAVE - 1);
#pragma unroll
    for (int i = 0; i < MAXD; ++i) acc[i] *= alpha;
    for (int j = first; j <= last; ++j) {
      const float pj = p_lds[j];
      const int rj = __shfl(row, j, PAE_WAVE);
      // values are transposed within a page: [block][kv head][feature][offset in page]
      const T* vr = v_cache + (int64_t)(rj / bs) * bs * hd + rj % bs;
#pragma unroll
      for (int i = 0; i < MAXD; ++i) {
        const int d = lane + i * PAE_WAVE;
        if (d < hd) acc[i] = fmaf(pj, to_f32(vr[(int64_t)d * bs]), acc[i]);
      }
    }
    __syncthreads();
  }
  T* o = out + (int64_t)t * out_stride + (int64_t)head * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = lane + i * PAE_WAVE;
    if (d < hd) o[d] = from_f32<T>(acc[i] * inv);
  }
}

template <typename T>
static int launch_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int* positions, const int* tok_seq,
                          const int* block_tables, int max_blocks, int bs, int num_tokens, int nh, int nkv,
                          int hd, float scale, int window, hipStream_t stream) {
  dim3 grid(num_tokens, nh);
  const size_t lds = (size_t)(hd + PAE_WAVE) * sizeof(float);
#define PAE_LAUNCH(MAXD)                                                                              \
  paged_attention_generic_kernel<T, MAXD><<<grid, PAE_WAVE, lds, stream>>>(                           \
      (T*)out, out_stride, (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, positions,    \
      tok_seq, block_tables, max_blocks, bs, nh, nkv, hd, scale, window)
  if (hd <= 64) PAE_LAUNCH(1);
  else if (hd <= 128) PAE_LAUNCH(2);
  else if (hd <= 192) PAE_LAUNCH(3);
  else PAE_LAUNCH(4);
#undef PAE_LAUNCH
  return pae_check_launch("paged_attention_generic");
}

extern "C" int pae_paged_attention_generic(int dtype, void* out, int64_t out_stride, const void* q,
                                           int64_t q_stride, const void* k_cache, const void* v_cache,
                                           const int* positions, const int* tok_seq,
                                           const int* block_tables, int max_blocks, int bs,
                                           int num_tokens, int nh, int nkv, int hd, float scale,
                                           int window, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attention: %d query heads over %d key/value heads", nh, nkv);
  PAE_REQUIRE(hd > 0 && hd <= 256, "attention: head_dim %d is outside 1..256", hd);
  PAE_REQUIRE(bs > 0 && max_blocks > 0, "attention: bad cache geometry bs=%d max_blocks=%d", bs, max_blocks);
  PAE_REQUIRE(window >= 0, "attention: negative window %d", window);
  PAE_REQUIRE(nh <= 65535, "attention: %d query heads exceed the grid", nh);
  if (num_tokens <= 0) return 0;
  if (dtype == PAE_F32)
    return launch_generic<float>(out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq,
                                 block_tables, max_blocks, bs, num_tokens, nh, nkv, hd, scale, window, stream);
  if (dtype == PAE_BF16)
    return launch_generic<bf16_t>(out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq,
                                  block_tables, max_blocks, bs, num_tokens, nh, nkv, hd, scale, window, stream);
  return pae_fail("attention: unknown dtype code %d", dtype);
}
