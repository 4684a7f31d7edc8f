// Device code shared by the few-row matrix products (gemm_skinny.hip) and the decode program
// (decode_program.hip): operand reordering for the matrix instruction, the epilogues (bias, rotation
// and cache write, SiLU gate, residual with the next norm's rows), the folded norm's row scales, and
// the sums of k ranges by ticket.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;

#define EPI_BF16 0
#define EPI_F32 1
#define EPI_SWIGLU 2
#define EPI_ROPE 3
#define EPI_RESIDUAL 4

// RMS normalisation folded into the products around it, so that a decode step needs no norm
// kernel between them.  norm(x) W^T = rsqrt(mean(x^2) + eps) * ((x * w_norm) W^T): the scale is one
// number per row and can be applied to the finished sums.
//
// Producer (EPI_RESIDUAL, the product that ends a residual branch): the sums of all k ranges are
// added into the float32 residual in place; the same tile is written again as
// bfloat16(residual * w_next), the rows the next product multiplies, and the tile's share of every
// row's sum of squares goes to next_stats[m][16-column tile].
// Consumer (any epilogue): `row_stats` holds those shares for the rows of A; every lane adds up
// its row's shares in a fixed order (the same in every workgroup, so all columns of a row get the
// same scale) and multiplies its sums by rsqrt(total / K + eps) before bias, rotation or gate.
struct SkinnyNorm {
  const float* row_stats;  // [M][row_stat_tiles] or null: A's rows are used as they are
  int row_stat_tiles;
  float eps;
  bf16_t* next_rows;       // EPI_RESIDUAL: [M][ld_next] bfloat16(residual * next_w)
  int64_t ld_next;
  const void* next_w;      // [N] weight of the norm that follows
  int next_w_is_f32;
  float* next_stats;       // [M][(N + 15) / 16]
};

// A pointer that a kernel has read from a description in LDS (not taken as a kernel argument) is a
// generic one to the compiler: loads through it are flat loads, which count on the LDS counter as well,
// so that every wait for an LDS read or a cross-lane permute would wait for all of them.  These tell the
// compiler that such a pointer points into device memory.
template <typename T>
__device__ __forceinline__ T* in_memory(T* p) {
  typedef T __attribute__((address_space(1))) InMemory;
  InMemory* g = (InMemory*)p;
  asm("" : "+v"(g));  // hides where it came from: the cast back is then known to come from device memory
  return (T*)g;
}
__device__ __forceinline__ const void* in_memory(const void* p) { return in_memory(reinterpret_cast<const char*>(p)); }
__device__ __forceinline__ void* in_memory(void* p) { return in_memory(reinterpret_cast<char*>(p)); }

// Loads that see what another die has written through during the same kernel (device-scope loads are
// served past the die's own L2, which may hold an older copy of the line); see `put` and SkinnyTickets below.
__device__ __forceinline__ float load_through(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 load_through(const f32x4* p) {
  unsigned long long raw[2];
  raw[0] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  raw[1] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return *reinterpret_cast<f32x4*>(raw);
}
__device__ __forceinline__ bf16x8 load_through(const bf16x8* p) {
  unsigned long long raw[2];
  raw[0] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  raw[1] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return *reinterpret_cast<bf16x8*>(raw);
}
__device__ __forceinline__ s16x4 load_through(const s16x4* p) {
  unsigned long long raw = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return *reinterpret_cast<s16x4*>(&raw);
}

// rsqrt(mean of squares + eps) of the rows of A from the shares the producer left, worked out once
// per workgroup by its first 256 threads together and left in LDS: PER_ROW threads to a row (16 for
// one column tile, 4 for more), each of which reads every PER_ROW-th group of four shares, all its
// reads in flight together (a thread that adds up a row in several trips to memory waits out the
// memory's latency once per trip: with eight trips a wavefront at the 7B width and 64 rows, 18 us a
// product), adds them in index order, and then the threads of a row add each other's in a fixed
// order.  The order depends on the width and on MT alone, so every workgroup of a product, and every
// kernel that takes one column tile, gives a row the same scale.
template <int MT>
struct ShareThreads {
  static constexpr int PER_ROW = MT == 1 ? 16 : 4;
  static constexpr int AT_ONCE = MT == 1 ? 8 : 16;  // groups of four shares a thread has in flight (up to 512 / 256 shares a row)
};

// The reads of thread t (0 .. 255 of the workgroup, or of a quad of wavefronts) from `base` on: row t / PER_ROW,
// the groups of four shares at base + 4 (PER_ROW u + t % PER_ROW), u < AT_ONCE.
template <int MT, int AT_ONCE, bool THROUGH>
struct RowShares {
  f32x4 part[AT_ONCE];
  __device__ __forceinline__ void ask(const SkinnyNorm& norm, int M, int t, int base) {
    constexpr int PER_ROW = ShareThreads<MT>::PER_ROW;
    const int m = t / PER_ROW, j = t % PER_ROW, tiles = norm.row_stat_tiles;
    const float* shares = norm.row_stats + (int64_t)(m < M ? m : M - 1) * tiles;
    // Rows of shares start on 16-byte boundaries where tiles % 4 == 0, and a group is then inside a row or
    // past it as a whole.  (Every group is zeroed first and loaded under one condition of its own: where two
    // branches load into the same registers the compiler waits for every load in flight in between.)
    if (tiles % 4 == 0) {
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u) {
        const int at = base + 4 * (PER_ROW * u + j);
        part[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (at < tiles)
          part[u] = THROUGH ? load_through(reinterpret_cast<const f32x4*>(shares + at)) : *reinterpret_cast<const f32x4*>(shares + at);
      }
    } else {
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u) {
        const int at = base + 4 * (PER_ROW * u + j);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          part[u][i] = 0.f;
          if (at + i < tiles) part[u][i] = THROUGH ? load_through(shares + at + i) : shares[at + i];
        }
      }
    }
  }
  // one group after the other onto `s`: the sum does not depend on how many groups a trip holds
  __device__ __forceinline__ float add_to(float s) const {
#pragma unroll
    for (int u = 0; u < AT_ONCE; ++u) s += (part[u][0] + part[u][1]) + (part[u][2] + part[u][3]);
    return s;
  }
};

// The scales into s_scale[16 MT] (1 without a folded norm).  Threads t >= 256 do nothing.  The
// caller puts a workgroup barrier between this and the first read of s_scale.  `before_sum`: called
// between asking and adding (the place for loads that should be on their way meanwhile).  AT_ONCE:
// the groups of a trip; fewer cost registers less and wide rows further trips, and give the same bits.
template <int MT, bool THROUGH = false, int AT_ONCE = ShareThreads<MT>::AT_ONCE, typename Between>
__device__ __forceinline__ void row_scales_to_lds(float* s_scale, const SkinnyNorm& norm, int M, int K, int t,
                                                  Between before_sum) {
  constexpr int PER_ROW = ShareThreads<MT>::PER_ROW;
  const bool mine = t < 16 * MT * PER_ROW;  // whole wavefronts: 256 threads with one or four column tiles
  if (!norm.row_stats) {
    before_sum();
    if (t < 16 * MT) s_scale[t] = 1.0f;
    return;
  }
  const int tiles = norm.row_stat_tiles;
  constexpr int SPAN = 4 * PER_ROW * AT_ONCE;  // shares of a row that its threads take at once
  RowShares<MT, AT_ONCE, THROUGH> first;
  if (mine) first.ask(norm, M, t, 0);
  before_sum();
  if (!mine) return;
  float sum = first.add_to(0.f);
  for (int base = SPAN; base < tiles; base += SPAN) {  // wider rows: further trips
    RowShares<MT, AT_ONCE, THROUGH> more;
    more.ask(norm, M, t, base);
    sum = more.add_to(sum);
  }
#pragma unroll
  for (int step = 1; step < PER_ROW; step *= 2) sum += __shfl_xor(sum, step);
  if (t % PER_ROW == 0) s_scale[t / PER_ROW] = rsqrtf(sum / (float)K + norm.eps);
}

// What the rotating epilogue needs beside the product: the head geometry, the
// rotation's frequencies, every row's position and sequence, and the paged cache.
struct SkinnyRope {
  const float* cos_sin;     // [M][rot / 2][2] cosine and sine of every row's angles, or null without rotation
  const int* positions;     // [M]
  const int* tok_seq;       // [M] row of block_tables
  const int* block_tables;  // [sequences][max_blocks]
  bf16_t* k_cache;          // [block][kv head][bs][hd]
  bf16_t* v_cache;          // [block][kv head][hd][bs]
  int nh, nkv, hd, rot, max_blocks, bs;
};

__device__ __forceinline__ SkinnyNorm in_memory(const SkinnyNorm& n) {
  return SkinnyNorm{in_memory(n.row_stats), n.row_stat_tiles, n.eps, in_memory(n.next_rows), n.ld_next,
                    in_memory(n.next_w), n.next_w_is_f32, in_memory(n.next_stats)};
}
__device__ __forceinline__ SkinnyRope in_memory(const SkinnyRope& r) {
  return SkinnyRope{in_memory(r.cos_sin), in_memory(r.positions), in_memory(r.tok_seq), in_memory(r.block_tables),
                    in_memory(r.k_cache), in_memory(r.v_cache), r.nh, r.nkv, r.hd, r.rot, r.max_blocks, r.bs};
}

// Feature within its head of row `r` of the `j`-th tile of a head: a tile inside the rotated
// part holds features 8 j .. 8 j + 7 (rows 0-7) and their partners rot / 2 + 8 j .. (rows 8-15);
// tiles past it hold 16 consecutive features that pass through.
__device__ __forceinline__ int rope_feature(int j, int r, int rot) {
  return 16 * j < rot ? (r < 8 ? 8 * j + r : rot / 2 + 8 * j + r - 8) : 16 * j + r;
}

// A fragment loaded as (row = lane / 4, k group = lane % 4) moved to (row = lane % 16, k group = lane / 16).
__device__ __forceinline__ bf16x8 to_mfma_order(bf16x8 v, int fetch_from) {
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  i32x4 raw = *reinterpret_cast<i32x4*>(&v);
#pragma unroll
  for (int i = 0; i < 4; ++i) raw[i] = __builtin_amdgcn_ds_bpermute(fetch_from, raw[i]);
  return *reinterpret_cast<bf16x8*>(&raw);
}

__device__ __forceinline__ short to_bf16_bits(float x) {
  const bf16_t h = __float2bfloat16(x);
  return *reinterpret_cast<const short*>(&h);
}

// Stores that the other dies of the chip can read once they have been acknowledged: device-scope
// stores are written through the die's own L2 to the memory side, where all dies agree (see
// SkinnyTickets below).  A kernel whose workgroups hand results to one another across a barrier of
// their own (decode_program.hip) stores everything it hands on this way; ordinary kernels, whose
// results are read by the next kernel, store plainly (THROUGH = false).
template <bool THROUGH>
__device__ __forceinline__ void put(s16x4* p, s16x4 v) {
  if (THROUGH) __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), *reinterpret_cast<unsigned long long*>(&v),
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}
template <bool THROUGH>
__device__ __forceinline__ void put(f32x4* p, f32x4 v) {
  if (THROUGH) {
    unsigned long long* raw = reinterpret_cast<unsigned long long*>(&v);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), raw[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p) + 1, raw[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else *p = v;
}
template <bool THROUGH>
__device__ __forceinline__ void put(float* p, float v) {
  if (THROUGH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}
template <bool THROUGH>
__device__ __forceinline__ void put(short* p, short v) {
  if (THROUGH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

// What an epilogue reads beside the sums (the residual's tile and the next norm's weights; a row's
// position, its page of the cache and its angles), asked for before the products are made, so that the
// trips to memory are over when the sums are there.  One column tile only (up to 16 rows of A).
template <int RT>
struct EpilogueAhead {
  float res[RT][4], next_w[RT][4];  // EPI_RESIDUAL
  int pos, seq;                     // EPI_ROPE: the row's position and its row of the block tables
  int64_t page;                     //   first element of the row's page in the pools
  float cs[RT][4][2];               //   cosine and sine of this lane's four features
};

// The part of it that belongs to the row of A alone, and that the page's number waits for: asked for
// first of all, so that it is there when ask_epilogue wants it.
template <int RT, int EPI>
__device__ __forceinline__ void ask_row(EpilogueAhead<RT>& pre, int M, const SkinnyRope& rope) {
  if (EPI == EPI_ROPE) {
    const int r = threadIdx.x % 16, mc = r < M ? r : M - 1;
    pre.pos = rope.positions[mc];
    pre.seq = rope.nkv > 0 ? rope.tok_seq[mc] : 0;  // (no table without key/value heads)
  }
}

// (after ask_row)
template <int RT, int EPI, bool THROUGH>
__device__ __forceinline__ void ask_epilogue(EpilogueAhead<RT>& pre, int tile_base, const void* out, int64_t ldc,
                                             int M, int N, const SkinnyRope& rope, const SkinnyNorm& norm) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int r = lane % 16, g4 = lane / 16;
  const int mc = r < M ? r : M - 1;
  if (EPI == EPI_RESIDUAL) {
    const float* res = (const float*)out + (int64_t)mc * ldc;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n = 16 * (tile_base + rt) + 4 * g4;
      if (!THROUGH && ldc % 4 == 0 && n + 4 <= N) {  // the same in the whole wavefront but for the last tile
        const f32x4 v = *reinterpret_cast<const f32x4*>(res + n);
#pragma unroll
        for (int i = 0; i < 4; ++i) pre.res[rt][i] = v[i];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int nc = n + i < N ? n + i : N - 1;
          pre.res[rt][i] = THROUGH ? load_through(res + nc) : res[nc];
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) pre.next_w[rt][i] = load_param(norm.next_w, norm.next_w_is_f32, n + i < N ? n + i : N - 1);
    }
  }
  if (EPI == EPI_ROPE) {
    const int per_head = rope.hd / 16;
    bool any_cache = false;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int tile = tile_base + rt, head = tile / per_head, j = tile % per_head;
      any_cache = any_cache || head >= rope.nh;
      const bool rotated = 16 * j < rope.rot && head < rope.nh + rope.nkv;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float* angle = rope.cos_sin + ((int64_t)mc * (rope.rot / 2) + 8 * j + (4 * g4 + i) % 8) * 2;
        pre.cs[rt][i][0] = rotated ? angle[0] : 1.f;
        pre.cs[rt][i][1] = rotated ? angle[1] : 0.f;
      }
    }
    pre.page = 0;
    if (any_cache)
      pre.page = (int64_t)rope.block_tables[(int64_t)pre.seq * rope.max_blocks + pre.pos / rope.bs] *
                 rope.nkv * ((int64_t)rope.bs * rope.hd);
  }
}

// What a wavefront does with finished sums: acc[rt][mt] is the 16 x 16 tile of weight rows
// 16 (tile_base + rt) .. (through the rotation's row order, if any) by rows 16 mt .. of A; a lane
// holds row m = 16 mt + lane % 16 of A and weight rows 4 (lane / 16) + i.  only_mt >= 0: just
// that column tile (the others belong to other wavefronts).
template <int MT, int RT, int EPI, bool THROUGH = false>
__device__ __forceinline__ void skinny_epilogue(const f32x4 (&acc)[RT][MT], int tile_base, int only_mt,
                                                void* __restrict__ out, int64_t ldc, const void* __restrict__ bias,
                                                int b_is_f32, int M, int N, int split, int64_t part_stride,
                                                const SkinnyRope& rope, const SkinnyNorm& norm,
                                                const float (&scale)[MT], const EpilogueAhead<RT>* pre = nullptr) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int r = lane % 16, g4 = lane / 16;
  if (EPI == EPI_ROPE) {
    // lane holds row m = 16 mt + r of A and rows 4 g4 + i of each tile: lanes 0-31 the lower
    // features of the pairs, lanes 32-63 (same m) their partners
    const int per_head = rope.hd / 16;
    const int64_t head_step = (int64_t)rope.bs * rope.hd;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (only_mt >= 0 && mt != only_mt) continue;  // another wavefront's column tile
      const int m = 16 * mt + r;
      const int mc = m < M ? m : M - 1;
      const int pos = pre ? pre->pos : rope.positions[mc];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int tile = tile_base + rt;
        const int head = tile / per_head, j = tile % per_head;
        const bool rotated = 16 * j < rope.rot && head < rope.nh + rope.nkv;  // values keep the tile layout, unrotated
        const int f0 = rope_feature(j, 4 * g4, rope.rot);  // first of this lane's 4 consecutive features
        const int n = head * rope.hd + f0;
        s16x4 res;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // the projection is rounded to bfloat16 before the rotation, as where the two are separate kernels
          const float own = __bfloat162float(__float2bfloat16(
              acc[rt][mt][i] * scale[mt] + ((bias && n + i < N) ? load_param(bias, b_is_f32, n + i) : 0.f)));
          const float other = __shfl_xor(own, 32);  // in every lane
          float o = own;
          if (rotated) {
            const float* angle = rope.cos_sin + ((int64_t)mc * (rope.rot / 2) + 8 * j + (4 * g4 + i) % 8) * 2;
            const float cs = pre ? pre->cs[rt][i][0] : angle[0], sn = pre ? pre->cs[rt][i][1] : angle[1];
            o = g4 < 2 ? own * cs - other * sn : own * cs + other * sn;
          }
          res[i] = to_bf16_bits(o);
        }
        if (m >= M || n >= N) continue;
        if (head < rope.nh) {
          put<THROUGH>(reinterpret_cast<s16x4*>((bf16_t*)out + (int64_t)m * ldc + n), res);
          continue;
        }
        const int off = pos % rope.bs;
        const int64_t page = pre ? pre->page
                                 : (int64_t)rope.block_tables[(int64_t)rope.tok_seq[m] * rope.max_blocks + pos / rope.bs] *
                                       rope.nkv * head_step;
        if (head < rope.nh + rope.nkv) {
          put<THROUGH>(reinterpret_cast<s16x4*>(rope.k_cache + page + (head - rope.nh) * head_step + (int64_t)off * rope.hd + f0), res);
        } else {
          short* dst = reinterpret_cast<short*>(rope.v_cache) + page + (head - rope.nh - rope.nkv) * head_step +
                       (int64_t)f0 * rope.bs + off;
#pragma unroll
          for (int i = 0; i < 4; ++i) put<THROUGH>(dst + (int64_t)i * rope.bs, res[i]);
        }
      }
    }
    return;
  }

  const bool vec = ldc % 4 == 0;  // rows of out keep 8- and 16-byte stores aligned
  // lane holds, per column tile mt, row m = 16 mt + r of A and weight rows 4 g4 + i of each row tile
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (only_mt >= 0 && mt != only_mt) continue;  // another wavefront's column tile
    const int m = 16 * mt + r;
    if (m >= M) continue;
    if (EPI == EPI_SWIGLU) {
      // a tile holds 8 gate rows (lanes 0-31: rows 4 g4 + i) and their 8 up rows (lanes 32-63, same m)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int j = (tile_base + rt) * 8 + 4 * (g4 % 2);  // output feature of register 0
        s16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float own = acc[rt][mt][i] * scale[mt];
          const float up = __shfl_xor(own, 32);  // in every lane (the same row of A, so the same scale)
          v[i] = to_bf16_bits(own / (1.0f + expf(-own)) * up);
        }
        if (g4 < 2 && j < N / 2)  // N counts gate and up rows
          put<THROUGH>(reinterpret_cast<s16x4*>((bf16_t*)out + (int64_t)m * ldc + j), v);
      }
    } else if (EPI == EPI_RESIDUAL) {
      // residual += sums; the next product's rows and this tile's share of the row's sum of squares
      float* res = (float*)out + (int64_t)m * ldc;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int n = 16 * (tile_base + rt) + 4 * g4;
        float ss = 0.f;
        if (n < N) {
          float v[4];
          s16x4 p;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool in = n + i < N;
            v[i] = in ? (pre ? pre->res[rt][i] : THROUGH ? load_through(res + n + i) : res[n + i]) + acc[rt][mt][i] * scale[mt] : 0.f;
            ss += v[i] * v[i];
            p[i] = to_bf16_bits(in ? v[i] * (pre ? pre->next_w[rt][i] : load_param(norm.next_w, norm.next_w_is_f32, n + i)) : 0.f);
          }
          bf16_t* nxt = norm.next_rows + (int64_t)m * norm.ld_next + n;
          if (vec && norm.ld_next % 4 == 0 && n + 4 <= N) {
            put<THROUGH>(reinterpret_cast<f32x4*>(res + n), (f32x4){v[0], v[1], v[2], v[3]});
            put<THROUGH>(reinterpret_cast<s16x4*>(nxt), p);
          } else {
            for (int i = 0; i < 4 && n + i < N; ++i) {
              put<THROUGH>(res + n + i, v[i]);
              put<THROUGH>(reinterpret_cast<short*>(nxt) + i, p[i]);
            }
          }
        }
        ss += __shfl_xor(ss, 16);  // the four lanes that hold this row's 16 columns
        ss += __shfl_xor(ss, 32);
        if (g4 == 0 && 16 * (tile_base + rt) < N)
          put<THROUGH>(norm.next_stats + (int64_t)m * ((N + 15) / 16) + tile_base + rt, ss);
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int n = 16 * (tile_base + rt) + 4 * g4;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] = acc[rt][mt][i] * scale[mt] + ((bias && n + i < N) ? load_param(bias, b_is_f32, n + i) : 0.f);
        if (EPI == EPI_F32) {
          float* dst = (float*)out + (int64_t)split * part_stride + (int64_t)m * ldc + n;
          if (vec && n + 4 <= N) put<THROUGH>(reinterpret_cast<f32x4*>(dst), (f32x4){v[0], v[1], v[2], v[3]});
          else
            for (int i = 0; i < 4 && n + i < N; ++i) put<THROUGH>(dst + i, v[i]);
        } else {
          bf16_t* dst = (bf16_t*)out + (int64_t)m * ldc + n;
          if (vec && n + 4 <= N) {
            s16x4 p;
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = to_bf16_bits(v[i]);
            put<THROUGH>(reinterpret_cast<s16x4*>(dst), p);
          } else
            for (int i = 0; i < 4 && n + i < N; ++i) put<THROUGH>(reinterpret_cast<short*>(dst) + i, to_bf16_bits(v[i]));
        }
      }
    }
  }
}

// Several k ranges for an epilogue that needs whole sums (bias, rotation, gate): every range's
// workgroup leaves its partial tile in `parts` and draws a ticket from the tile's counter; the one
// that draws the last ticket knows that all partials are written, adds them in range order
// whichever workgroup it is (so the sums do not depend on the order of arrival), puts the counter
// back to zero and runs the epilogue.  Nobody waits for anybody.
//
// Why relaxed device-scope atomics and one wait are enough here (gfx942/gfx950).  The chip is eight
// dies, each with an L2 of its own that is not kept coherent with the others'; the memory side behind
// them (the shared last-level cache and HBM) is the point at which all dies agree.  A device-scope
// ("agent") atomic store or load is issued with the sc1 bit: the store is written through to that
// point and the load is served from it, whatever either die's L2 holds.  `s_waitcnt vmcnt(0)` returns
// when every vector memory operation of the wavefront, these stores included, has been
// acknowledged, which for a written-through store means that it has arrived there.  So: (1) a
// workgroup's partial sums are at the common point before it draws its ticket; (2) the ticket is a
// device-scope read-modify-write, carried out at the same point, so tickets are handed out in one
// order, and whoever draws the last one does so after every other range's partials have arrived;
// (3) its loads of the partials are issued after the ticket's value has come back (they sit behind a
// branch on that value and a compiler barrier) and, being sc1 loads, cannot be served stale from a
// cache.  A release fence would add a write-back of the die's whole L2 (`buffer_wbl2`) for the sake
// of ordinary stores that may still be dirty there; there are none that matter, because the
// partials never were ordinary stores (measured: 13 us a launch with the fence, 1 us without).
// The counters are shared by every launch on a device: the launches must not overlap, which the
// host side enforces by tying the counters to one stream.
struct SkinnyTickets {
  float* parts;   // [slots][k ranges][RT * 4][64]: a wavefront's accumulators, lane by lane
  int* counters;  // [slots], zero before and after every launch; null: one k range
};

// True in the wavefront that holds the whole sums afterwards (in `acc`); the others are done.
template <int RT, int AT_ONCE = (RT == 1 ? 8 : RT == 2 ? 4 : 2)>
__device__ __forceinline__ bool add_up_k_ranges(f32x4 (&acc)[RT], int slot, int split, int splits,
                                                const SkinnyTickets& tk) {
  const int lane = threadIdx.x % PAE_WAVE;
  float* mine = tk.parts + ((int64_t)slot * splits + split) * (RT * 4 * PAE_WAVE) + lane;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __hip_atomic_store(mine + (rt * 4 + i) * PAE_WAVE, acc[rt][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every lane's stores have arrived
  int ticket = 0;
  if (lane == 0) ticket = __hip_atomic_fetch_add(tk.counters + slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  ticket = __builtin_amdgcn_readfirstlane(ticket);
  asm volatile("" ::: "memory");
  if (ticket != splits - 1) return false;  // the same in every lane
  if (lane == 0) __hip_atomic_store(tk.counters + slot, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // added in range order; the loads of AT_ONCE ranges are in flight together (one after the other, every
  // range would wait out a trip to memory of its own: 32 registers by default, which the products' loops
  // have left free by now, 64 with eight tiles)
  for (int p0 = 0; p0 < splits; p0 += AT_ONCE) {
    float theirs[AT_ONCE][RT * 4];
#pragma unroll
    for (int q = 0; q < AT_ONCE; ++q) {
      const int p = p0 + q < splits ? p0 + q : splits - 1;  // past the last range: loaded again, not added
      const float* from = tk.parts + ((int64_t)slot * splits + p) * (RT * 4 * PAE_WAVE) + lane;
#pragma unroll
      for (int j = 0; j < RT * 4; ++j)
        theirs[q][j] = __hip_atomic_load(from + j * PAE_WAVE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int q = 0; q < AT_ONCE; ++q) {
      if (p0 + q >= splits) break;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][i] += theirs[q][rt * 4 + i];
    }
  }
  return true;
}

