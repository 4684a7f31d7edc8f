// Row-wise kernels around the matrix products: embedding gather, residual add
// fused with RMS normalisation, rotary position encoding fused with the write of
// keys and values into their cache pages, and the SiLU gate of the feed-forward.
//
// The residual stream is float32 in both precisions; T is the storage type of
// activations that feed matrix products (float or bfloat16).  Sums of squares,
// rotation angles and the gate are computed in float32 and rounded once.
#include "common.h"
#include "api.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = scale * table[ids[t], :]  (engine/model.py:401,448 of the reference: a plain
// row gather; its model has no scaling, so scale is 1 there and the product is exact)
template <typename T>
__global__ void embedding_kernel(float* __restrict__ out, const T* __restrict__ table,
                                 const int* __restrict__ ids, int hidden, float scale) {
  const int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * hidden;
  float* dst = out + (int64_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = scale * to_f32(row[i]);
}

extern "C" int pae_embedding(int dtype, void* out, const void* table, const int* ids, int num_tokens,
                             int hidden, int vocab, float scale, hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes T=%d H=%d V=%d",
              num_tokens, hidden, vocab);
  if (num_tokens == 0) return 0;
  if (dtype == PAE_F32)
    embedding_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)out, (const float*)table, ids, hidden, scale);
  else if (dtype == PAE_BF16)
    embedding_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((float*)out, (const bf16_t*)table, ids, hidden, scale);
  else
    return pae_fail("embedding: unknown dtype code %d", dtype);
  return pae_check_launch("embedding");
}

// The embedding for a step whose first norm is folded into the products around it (see
// gemm_skinny.hip): beside the float32 rows, bfloat16(row * next_w) for the first product and the
// shares of every row's sum of squares, one per 16 columns.
template <typename T>
__global__ void embedding_rows_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids,
                                      int hidden, float scale, bf16_t* __restrict__ next_rows,
                                      const void* __restrict__ next_w, int next_w_is_f32,
                                      float* __restrict__ next_stats) {
  // four lanes to a tile of 16 columns, four columns each; their squares meet through two shuffles
  const int t = blockIdx.x, tiles = (hidden + 15) / 16;
  const T* row = table + (int64_t)ids[t] * hidden;
  const int quarter = threadIdx.x % 4;
  for (int tile = threadIdx.x / 4; tile < (tiles + 63) / 64 * 64; tile += blockDim.x / 4) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = 16 * tile + 4 * quarter + j;
      if (tile < tiles && i < hidden) {
        const float v = scale * to_f32(row[i]);
        out[(int64_t)t * hidden + i] = v;
        next_rows[(int64_t)t * hidden + i] = __float2bfloat16(v * load_param(next_w, next_w_is_f32, i));
        ss += v * v;
      }
    }
    ss += __shfl_xor(ss, 1);
    ss += __shfl_xor(ss, 2);
    if (quarter == 0 && tile < tiles) next_stats[(int64_t)t * tiles + tile] = ss;
  }
}

extern "C" int pae_embedding_rows(int dtype, void* residual, const void* table, const int* ids, int num_tokens,
                                  int hidden, int vocab, float scale, void* next_rows, const void* next_w,
                                  int next_w_is_f32, float* next_stats, hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0, "embedding_rows: bad sizes T=%d H=%d V=%d", num_tokens, hidden, vocab);
  PAE_REQUIRE(next_rows && next_w && next_stats, "embedding_rows: the next product's rows, weight and sums are missing");
  if (num_tokens == 0) return 0;
  if (dtype == PAE_F32)
    embedding_rows_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)residual, (const float*)table, ids, hidden, scale,
                                                                 (bf16_t*)next_rows, next_w, next_w_is_f32, next_stats);
  else if (dtype == PAE_BF16)
    embedding_rows_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((float*)residual, (const bf16_t*)table, ids, hidden, scale,
                                                                  (bf16_t*)next_rows, next_w, next_w_is_f32, next_stats);
  else
    return pae_fail("embedding_rows: unknown dtype code %d", dtype);
  return pae_check_launch("embedding_rows");
}

// out[m] = bfloat16(rows[m] * rsqrt(sum(row_stats[m]) / hidden + eps)): rows whose scale is still
// owed (see gemm_skinny.hip), paid here for a part that wants plain normalised activations.  The
// shares are added in the order the products add them.
__global__ void scaled_rows_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ rows,
                                   const float* __restrict__ row_stats, int tiles, float eps, int hidden) {
  __shared__ float s_scale;
  const int m = blockIdx.x;
  if (threadIdx.x < PAE_WAVE) {
    // the order in which the products of up to 16 rows add the shares (skinny_device.h, row_scales_to_lds):
    // sixteen threads a row, thread j the groups of four at 4 (16 u + j), one after the other
    const int j = threadIdx.x % 16;
    const float* shares = row_stats + (int64_t)m * tiles;
    float sum = 0.f;
    for (int t = 4 * j; t < tiles; t += 64) {
      float v[4];
      for (int i = 0; i < 4; ++i) v[i] = t + i < tiles ? shares[t + i] : 0.f;
      sum += (v[0] + v[1]) + (v[2] + v[3]);
    }
    for (int step = 1; step < 16; step *= 2) sum += __shfl_xor(sum, step);
    if (threadIdx.x == 0) s_scale = rsqrtf(sum / (float)hidden + eps);
  }
  __syncthreads();
  const float scale = s_scale;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    out[(int64_t)m * hidden + i] = __float2bfloat16(__bfloat162float(rows[(int64_t)m * hidden + i]) * scale);
}

extern "C" int pae_scaled_rows(void* out, const void* rows, const float* row_stats, int row_stat_tiles, float eps,
                               int num_rows, int hidden, hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && hidden > 0 && row_stat_tiles > 0 && row_stats, "scaled_rows: bad sizes rows=%d H=%d tiles=%d",
              num_rows, hidden, row_stat_tiles);
  if (num_rows == 0) return 0;
  scaled_rows_kernel<<<num_rows, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)rows, row_stats, row_stat_tiles, eps, hidden);
  return pae_check_launch("scaled_rows");
}

// ---------------------------------------------------------------- logits: scale and soft cap
// x = scale * x, then, with cap > 0, x = cap * tanh(x / cap).  Not part of the reference's model
// (its logits are the head product as it is); an architecture's plan may ask for either.
__global__ void logits_finish_kernel(float* __restrict__ x, int64_t n, float scale, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = scale * x[i];
  if (cap > 0.f) v = cap * tanhf(v / cap);
  x[i] = v;
}

extern "C" int pae_logits_finish(float* logits, int64_t n, float scale, float cap, hipStream_t stream) {
  PAE_REQUIRE(n >= 0 && n <= ((int64_t)1 << 38), "logits_finish: bad count %lld", (long long)n);
  PAE_REQUIRE(cap >= 0.f, "logits_finish: the soft cap %g must not be negative (0 switches it off)", (double)cap);
  if (n == 0) return 0;
  logits_finish_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(logits, n, scale, cap);
  return pae_check_launch("logits_finish");
}

// ---------------------------------------------------------------- add + RMSNorm
// r = residual[row] (+ delta[row]);  residual[row] = r if write_residual;
// out[b] = weight * T(r * rsqrt(mean(r^2) + eps))
// The normalised value is rounded to T before the weight multiply, as the
// reference does (engine/model.py:117-123: float32 inside, cast back, then scale).
// With `rows` given, block b reads source row rows[b] (gather of selected rows).
// The pending branch output `delta` is either in the storage type T (parts == 0) or
// `parts` float32 partial sums, `part_stride` elements apart, added in order.
template <typename T>
__device__ __forceinline__ float pending_at(const void* delta, int parts, int64_t part_stride, int64_t idx) {
  if (parts == 0) return to_f32(((const T*)delta)[idx]);
  float sum = 0.f;
  for (int p = 0; p < parts; ++p) sum += ((const float*)delta)[p * part_stride + idx];
  return sum;
}

// Sum over the wavefronts of a block of any size, in wavefront order.
__device__ __forceinline__ float block_sum_any(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / PAE_WAVE, nwaves = (blockDim.x + PAE_WAVE - 1) / PAE_WAVE;
  if ((threadIdx.x & (PAE_WAVE - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  __syncthreads();
  return total;
}

template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
  typedef float4 type;
  static __device__ __forceinline__ void unpack(const type& v, float (&f)[4]) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
  static __device__ __forceinline__ type pack(const float (&f)[4]) { return make_float4(f[0], f[1], f[2], f[3]); }
};
template <>
struct Vec4<bf16_t> {
  typedef uint2 type;  // four bfloat16
  static __device__ __forceinline__ void unpack(const type& v, float (&f)[4]) {
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ type pack(const float (&f)[4]) {
    bf16_t h[4] = {__float2bfloat16(f[0]), __float2bfloat16(f[1]), __float2bfloat16(f[2]), __float2bfloat16(f[3])};
    return *reinterpret_cast<const type*>(h);
  }
};

// Vector form for hidden % 4 == 0: a thread owns chunks of four elements; the launch
// gives one chunk per thread up to a width of 4096, so a row is one round of loads.
// The kernel is kept small on purpose: at a few rows it runs for microseconds and the
// time goes to fetching its instructions.
template <typename T>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ residual, const void* __restrict__ delta, int parts,
                                       int64_t part_stride, const void* __restrict__ weight, int w_is_f32,
                                       float eps, const int* __restrict__ rows, T* __restrict__ out, int hidden,
                                       int write_residual) {
  __shared__ float scratch[16];
  typedef typename Vec4<T>::type vec_t;
  const int b = blockIdx.x;
  const int64_t src = rows ? rows[b] : b;
  const int nvec = hidden / 4;
  float4* res4 = reinterpret_cast<float4*>(residual + src * hidden);
  const bool one_round = nvec <= (int)blockDim.x;  // every thread has at most one chunk: keep it in registers
  float ss = 0.f;
  float4 mine = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int v = threadIdx.x; v < nvec; v += blockDim.x) {
    float4 r = res4[v];
    if (delta) {
      if (parts == 0) {
        float d[4];
        Vec4<T>::unpack(reinterpret_cast<const vec_t*>((const T*)delta + src * hidden)[v], d);
        r.x += d[0]; r.y += d[1]; r.z += d[2]; r.w += d[3];
      } else {
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);  // partial sums are added in order
        for (int p = 0; p < parts; ++p) {
          const float4 d = reinterpret_cast<const float4*>((const float*)delta + p * part_stride + src * hidden)[v];
          sum.x += d.x; sum.y += d.y; sum.z += d.z; sum.w += d.w;
        }
        r.x += sum.x; r.y += sum.y; r.z += sum.z; r.w += sum.w;
      }
      if (write_residual) res4[v] = r;
    }
    ss += (r.x * r.x + r.y * r.y) + (r.z * r.z + r.w * r.w);
    mine = r;
  }
  const float total = block_sum_any(ss, scratch);  // every thread of the block arrives here together
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  for (int v = threadIdx.x; v < nvec; v += blockDim.x) {
    float4 r = mine;
    if (!one_round) {
      r = res4[v];
      if (delta && !write_residual)
        for (int i = 0; i < 4; ++i) (&r.x)[i] += pending_at<T>(delta, parts, part_stride, src * hidden + 4 * v + i);
    }
    float w[4], o[4] = {r.x, r.y, r.z, r.w};
    if (w_is_f32) {
      const float4 wv = reinterpret_cast<const float4*>(weight)[v];
      w[0] = wv.x; w[1] = wv.y; w[2] = wv.z; w[3] = wv.w;
    } else {
      Vec4<bf16_t>::unpack(reinterpret_cast<const uint2*>(weight)[v], w);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = w[i] * round_to<T>(o[i] * inv);
    reinterpret_cast<vec_t*>(out + (int64_t)b * hidden)[v] = Vec4<T>::pack(o);
  }
}

// Any width, two passes over the row.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void add_rmsnorm_kernel(float* __restrict__ residual,
                                                         const void* __restrict__ delta, int parts,
                                                         int64_t part_stride, const void* __restrict__ weight,
                                                         int w_is_f32, float eps, const int* __restrict__ rows,
                                                         T* __restrict__ out, int hidden, int write_residual) {
  __shared__ float scratch[NT / PAE_WAVE];
  const int b = blockIdx.x;
  const int64_t src = rows ? rows[b] : b;
  float* res = residual + src * hidden;
  T* dst = out + (int64_t)b * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += NT) {
    float r = res[i];
    if (delta) r += pending_at<T>(delta, parts, part_stride, src * hidden + i);
    if (write_residual && delta) res[i] = r;
    ss += r * r;
  }
  const float total = block_sum<NT / PAE_WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += NT) {
    float r = res[i];
    if (delta && !write_residual) r += pending_at<T>(delta, parts, part_stride, src * hidden + i);
    const float normed = round_to<T>(r * inv);
    dst[i] = from_f32<T>(load_param(weight, w_is_f32, i) * normed);
  }
}

extern "C" int pae_add_rmsnorm(int dtype, void* residual, const void* delta, int parts, int64_t part_stride,
                               const void* weight, int w_is_f32, float eps, const int* rows, void* out,
                               int num_rows, int hidden, int write_residual, hipStream_t stream) {
  PAE_REQUIRE(parts >= 0, "add_rmsnorm: negative number of partial sums");
  PAE_REQUIRE(num_rows >= 0 && hidden > 0, "add_rmsnorm: bad sizes rows=%d H=%d", num_rows, hidden);
  PAE_REQUIRE(!(rows && write_residual), "add_rmsnorm: a row gather may not write the residual back");
  if (num_rows == 0) return 0;
  const bool vec = hidden % 4 == 0;
  int threads = ((hidden / 4 + PAE_WAVE - 1) / PAE_WAVE) * PAE_WAVE;
  threads = threads > 1024 ? 1024 : threads;
#define RMS_LAUNCH(T)                                                                                         \
  if (vec)                                                                                                    \
    add_rmsnorm_vec_kernel<T><<<num_rows, threads, 0, stream>>>((float*)residual, delta, parts, part_stride,  \
                                                                weight, w_is_f32, eps, rows, (T*)out, hidden, \
                                                                write_residual);                              \
  else                                                                                                        \
    add_rmsnorm_kernel<T, 256><<<num_rows, 256, 0, stream>>>((float*)residual, delta, parts, part_stride,     \
                                                             weight, w_is_f32, eps, rows, (T*)out, hidden,    \
                                                             write_residual)
  if (dtype == PAE_F32) {
    RMS_LAUNCH(float);
  } else if (dtype == PAE_BF16) {
    RMS_LAUNCH(bf16_t);
  } else {
    return pae_fail("add_rmsnorm: unknown dtype code %d", dtype);
  }
#undef RMS_LAUNCH
  return pae_check_launch("add_rmsnorm");
}

// ---------------------------------------------------------------- residual add alone
// residual += delta (used when a block's output is needed without a following norm)
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ residual, const T* __restrict__ delta, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) residual[i] += to_f32(delta[i]);
}

extern "C" int pae_residual_add(int dtype, void* residual, const void* delta, int64_t n, hipStream_t stream) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == PAE_F32)
    residual_add_kernel<float><<<blocks, 256, 0, stream>>>((float*)residual, (const float*)delta, n);
  else if (dtype == PAE_BF16)
    residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>((float*)residual, (const bf16_t*)delta, n);
  else
    return pae_fail("residual_add: unknown dtype code %d", dtype);
  return pae_check_launch("residual_add");
}

// ---------------------------------------------------------------- token ids that are still on the device
// dst[dst_idx[i]] = src[src_idx[i]]: a step whose input token was sampled by the step before takes
// it from that step's output without a round trip through the host.
__global__ void scatter_i32_kernel(int* __restrict__ dst, const int* __restrict__ dst_idx,
                                   const int* __restrict__ src, const int* __restrict__ src_idx, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[dst_idx[i]] = src[src_idx[i]];
}

extern "C" int pae_scatter_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n,
                               hipStream_t stream) {
  PAE_REQUIRE(n >= 0, "scatter_i32: n=%d", n);
  if (n == 0) return 0;
  scatter_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, dst_idx, src, src_idx, n);
  return pae_check_launch("scatter_i32");
}

// dst[i] = src[i].  `src` may be pinned host memory, which the GPU reads over the bus: a step's few
// kilobytes of metadata reach the device by this kernel, in line with the kernels that need them,
// instead of through the copy engine, whose hand-over from and to the compute queue leaves the
// GPU idle for a few hundred microseconds between steps.
__global__ void copy_i32_kernel(int* __restrict__ dst, const int* __restrict__ src, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

extern "C" int pae_copy_i32(int* dst, const int* src, int n, hipStream_t stream) {
  PAE_REQUIRE(n >= 0 && dst && src, "copy_i32: n=%d", n);
  if (n == 0) return 0;
  copy_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, src, n);
  return pae_check_launch("copy_i32");
}

// ---------------------------------------------------------------- rotation + cache write
// qkv row t holds [q heads | k heads | v heads], each head `hd` wide.  Query and
// key heads are rotated over their first `rot` features in pairs (i, i + rot/2):
//   out[i]         = x[i] * cos - x[i + rot/2] * sin
//   out[i + rot/2] = x[i + rot/2] * cos + x[i] * sin
// with angle = position * inv_freq[i] in float32 (engine/model.py:126-161 of the
// reference; rotation after the bias, before the cache write, so the cache holds
// rotated keys and raw values).  Queries are rotated in place; keys and values
// go to slot block_table[seq][pos / bs] * bs + pos % bs of the cache
// (engine/attention.py:374-385,409-410); keys are laid out [block][kv head][bs][hd],
// values transposed within the page, [block][kv head][hd][bs].
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int64_t row_stride, int nh, int nkv, int hd,
                                     int rot, const void* __restrict__ bias, int b_is_f32,
                                     const float* __restrict__ cos_sin,
                                     const int* __restrict__ positions, const int* __restrict__ tok_seq,
                                     const int* __restrict__ block_tables, int max_blocks, int bs,
                                     T* __restrict__ k_cache, T* __restrict__ v_cache, int write_kv) {
  // One item per (head, rotated pair), then per (kv head, value feature): every thread's
  // loads are independent of the others' stores, so a token is one round of memory traffic.
  const int t = blockIdx.x;
  const int pos = positions[t];
  T* row = qkv + (int64_t)t * row_stride;
  int64_t page_base = 0;  // element offset of (block, kv head 0) in either pool
  const int64_t head_step = (int64_t)bs * hd;
  const int off = pos % bs;
  if (write_kv) page_base = (int64_t)block_tables[(int64_t)tok_seq[t] * max_blocks + pos / bs] * nkv * head_step;
  const int half = rot / 2;
  const int rotated_heads = nh + (write_kv ? nkv : 0);
  // with a bias, row[j] stands for round(row[j] + bias[j]): the projection's bias is added here, on
  // the way, where the product before left it out (the sum is rounded to T before the rotation, as
  // the projection's own bias epilogue would have rounded it)
  auto at = [&](int j) { return bias ? round_to<T>(to_f32(row[j]) + load_param(bias, b_is_f32, j)) : to_f32(row[j]); };
  for (int idx = threadIdx.x; idx < rotated_heads * half; idx += blockDim.x) {
    const int h = idx / half, i = idx % half;
    const float c = cos_sin[((int64_t)t * half + i) * 2], s = cos_sin[((int64_t)t * half + i) * 2 + 1];
    const float a = at(h * hd + i), b = at(h * hd + i + half);
    const T lo = from_f32<T>(a * c - b * s), hi = from_f32<T>(b * c + a * s);
    if (h < nh) {  // queries are rotated in place
      row[h * hd + i] = lo;
      row[h * hd + i + half] = hi;
    } else {       // keys go to [block][kv head][offset][feature]
      T* dst = k_cache + page_base + (h - nh) * head_step + (int64_t)off * hd;
      dst[i] = lo;
      dst[i + half] = hi;
    }
  }
  const int tail = hd - rot;  // features beyond the rotated ones pass through
  if (bias)  // ... but for the bias, which the queries' unrotated features still have to get
    for (int idx = threadIdx.x; idx < nh * tail; idx += blockDim.x) {
      const int j = (idx / tail) * hd + rot + idx % tail;
      row[j] = from_f32<T>(at(j));
    }
  if (!write_kv) return;
  for (int idx = threadIdx.x; idx < nkv * tail; idx += blockDim.x) {
    const int h = idx / tail, i = rot + idx % tail;
    k_cache[page_base + h * head_step + (int64_t)off * hd + i] = from_f32<T>(at((nh + h) * hd + i));
  }
  // values are stored transposed within a page: [block][kv head][feature][offset]
  for (int idx = threadIdx.x; idx < nkv * hd; idx += blockDim.x) {
    const int h = idx / hd, i = idx % hd;
    v_cache[page_base + h * head_step + (int64_t)i * bs + off] = from_f32<T>(at((nh + nkv + h) * hd + i));
  }
}

// cos_sin[t][i] = (cos, sin)(positions[t] * inv_freq[i]) for i < half: computed once per step and
// shared by every layer with the same rotation (angles in float32: engine/model.py:138-152).
__global__ void rope_table_kernel(float* __restrict__ cos_sin, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int half, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float s, c;
  sincosf((float)positions[idx / half] * inv_freq[idx % half], &s, &c);
  cos_sin[idx * 2] = c;
  cos_sin[idx * 2 + 1] = s;
}

extern "C" int pae_rope_table(float* cos_sin, const int* positions, const float* inv_freq, int num_tokens, int half,
                              hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && half > 0, "rope_table: bad sizes T=%d half=%d", num_tokens, half);
  const int64_t total = (int64_t)num_tokens * half;
  if (total == 0) return 0;
  rope_table_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(cos_sin, positions, inv_freq, half, total);
  return pae_check_launch("rope_table");
}

extern "C" int pae_rope_kv_write(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nh, int nkv,
                                 int hd, int rot, const void* bias, int b_is_f32, const float* cos_sin,
                                 const int* positions,
                                 const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                                 void* k_cache, void* v_cache, int write_kv, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv >= 0 && hd > 0, "rope_kv_write: bad head sizes nh=%d nkv=%d hd=%d", nh, nkv, hd);
  PAE_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotary_dim %d must be even and <= head_dim %d", rot, hd);
  PAE_REQUIRE(rot == 0 || cos_sin, "rope_kv_write: a rotation needs its table of cosines and sines");
  PAE_REQUIRE(row_stride >= (int64_t)(nh + 2 * nkv) * hd, "rope_kv_write: row stride %lld too small", (long long)row_stride);
  PAE_REQUIRE(!write_kv || (bs > 0 && max_blocks > 0 && k_cache && v_cache && block_tables && tok_seq),
              "rope_kv_write: cache write needs tables and pools");
  if (num_tokens <= 0) return 0;
  if (dtype == PAE_F32)
    rope_kv_write_kernel<float><<<num_tokens, 256, 0, stream>>>(
        (float*)qkv, row_stride, nh, nkv, hd, rot, bias, b_is_f32, cos_sin, positions, tok_seq, block_tables,
        max_blocks, bs, (float*)k_cache, (float*)v_cache, write_kv);
  else if (dtype == PAE_BF16)
    rope_kv_write_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, nh, nkv, hd, rot, bias, b_is_f32, cos_sin, positions, tok_seq, block_tables,
        max_blocks, bs, (bf16_t*)k_cache, (bf16_t*)v_cache, write_kv);
  else
    return pae_fail("rope_kv_write: unknown dtype code %d", dtype);
  return pae_check_launch("rope_kv_write");
}

// ---------------------------------------------------------------- SiLU gate
// out[t, j] = silu(x[t, j]) * x[t, inter + j],  silu(g) = g * sigmoid(g)
// (engine/model.py:317-320 of the reference; gate and up are the two halves of
// one fused projection here)
// With `block` > 0 the row holds blocks of `block` gate features followed by their
// `block` up features (the layout the skinny product's gated epilogue reads).
template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ x, int inter, int block, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / inter;
  const int j = (int)(idx % inter);
  const int64_t gi = block ? (int64_t)(j / block) * 2 * block + j % block : j;
  const int64_t ui = block ? gi + block : (int64_t)inter + j;
  const float g = to_f32(x[t * 2 * inter + gi]);
  const float u = to_f32(x[t * 2 * inter + ui]);
  out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

// Eight bfloat16 outputs per thread (16-byte loads and stores): used when the width and
// the block size are multiples of 8.
__global__ void swiglu_vec8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, int inter, int block,
                                   int64_t total_vecs) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_vecs) return;
  const int per_row = inter / 8;
  const int64_t t = idx / per_row;
  const int j = (int)(idx % per_row) * 8;
  const int64_t gi = block ? (int64_t)(j / block) * 2 * block + j % block : j;
  const int64_t ui = block ? gi + block : (int64_t)inter + j;
  const uint4 g4 = *reinterpret_cast<const uint4*>(x + t * 2 * inter + gi);
  const uint4 u4 = *reinterpret_cast<const uint4*>(x + t * 2 * inter + ui);
  const unsigned gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  unsigned ow[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
    const bf16_t o0 = __float2bfloat16(g0 / (1.0f + expf(-g0)) * u0);
    const bf16_t o1 = __float2bfloat16(g1 / (1.0f + expf(-g1)) * u1);
    ow[k] = (unsigned)(*reinterpret_cast<const unsigned short*>(&o0)) |
            ((unsigned)(*reinterpret_cast<const unsigned short*>(&o1)) << 16);
  }
  *reinterpret_cast<uint4*>(out + t * inter + j) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int pae_swiglu(int dtype, void* out, const void* x, int num_tokens, int inter, int block,
                          hipStream_t stream) {
  PAE_REQUIRE(num_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", num_tokens, inter);
  PAE_REQUIRE(block >= 0 && (block == 0 || inter % block == 0), "swiglu: blocks of %d do not divide %d", block, inter);
  const int64_t total = (int64_t)num_tokens * inter;
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == PAE_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)x, inter, block, total);
  else if (dtype == PAE_BF16) {
    if (inter % 8 == 0 && block % 8 == 0)
      swiglu_vec8_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x,
                                                                                 inter, block, total / 8);
    else
      swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, inter, block, total);
  } else
    return pae_fail("swiglu: unknown dtype code %d", dtype);
  return pae_check_launch("swiglu");
}
