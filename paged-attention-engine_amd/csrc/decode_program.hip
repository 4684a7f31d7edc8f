// A decode step's layers as one resident kernel.
//
// A step in which every sequence brings one token is a chain of short dependent kernels: per
// layer the query/key/value product, the split attention and its merge, the output product, the
// gated product and the down product.  Each of them moves a few megabytes and costs 4 to 7 us
// however little it moves, because a kernel boundary drains the chip and the next kernel's first
// loads wait out the memory's latency.  Here the chain is a list of phases that one kernel walks:
// as many workgroups as compute units stay resident for the whole step (512 threads each, two
// "quads" of four wavefronts) and meet at a barrier of their own between phases.
//
// Phases are the existing kernels' work, cut into items that the quads take in turn:
//   product    one item = 16 weight rows x one k range, the quad's wavefronts taking 32-wide k
//              steps in turn exactly as gemm_skinny_kernel<1, 1, EPI, 4> does (the same sums in the
//              same order, bit for bit), k ranges added up by ticket, any of that kernel's epilogues;
//   attention  one item = (token, key/value head, split of 128 keys) as attn_decode_kernel;
//   merge      one item = 64 (head, four features) of a (token, key/value head): its splits' partial
//              results added in attn_decode_merge_kernel's order, four groups of splits.
//
// What one workgroup writes and another reads after the barrier is written through to the memory
// side with device-scope stores (the dies' L2s are not coherent with one another, see
// skinny_device.h), acknowledged before the workgroup arrives at the barrier, and read with
// device-scope loads, which are served past the reader's own L2.  So that those loads stay few, a
// product's activations are read once per workgroup, into LDS.  Weights, tables and the cache's older
// pages, which nobody writes during the step, are read plainly.  Every pointer of a phase's description
// is passed through in_memory() where it is used: the description lives in LDS, and loads through a
// pointer read from there would otherwise be flat ones.  Every wait is bounded: a workgroup that
// has polled `spin_limit` times gives up, leaves an error code for the host and for the other
// workgroups, and the kernel ends.
#include "common.h"
#include "api.h"
#include "skinny_device.h"
#include "attention_device.h"
#include <type_traits>

#define PROG_PRODUCT 1
#define PROG_ATTENTION 2
#define PROG_MERGE 3
#ifndef PROG_QUADS
#define PROG_QUADS 2
#endif
#define PROG_THREADS (PROG_QUADS * 4 * PAE_WAVE)
#define PROG_MAX_ROWS 16
#define PROG_SPLIT 128    // keys per split of the attention phase: pae_attn_decode_split()
#define PROG_STAMPS 8        // numbers a workgroup may leave per phase in a trace (see pae_program_run)

struct ProgPhase {
  int type, epilogue;
  // product: out[M, N] (+)= A[M, K] W[N, K]^T through the epilogue
  int M, N, K, splits, k_per_split, b_is_f32;
  const bf16_t* W;
  const void* bias;
  const bf16_t* A;
  void* out;
  int64_t lda, ldc;
  SkinnyNorm norm;
  SkinnyRope rope;
  float* ticket_parts;
  int* ticket_counters;
  // decode attention
  const int4* dec_work;
  const int* block_tables;
  const bf16_t* q;
  bf16_t* attn_out;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  float* part_acc;
  float* part_ml;
  int64_t q_stride, out_stride;
  int num_dec, max_splits, max_blocks, bs, nh, nkv, hd, window;
  float scale_log2;
  int pad_[3];
};
static_assert(sizeof(ProgPhase) % 16 == 0, "phases are copied as 16-byte pieces");

// A barrier across the workgroups in two levels.  Arrivals are counted in one counter per die (the
// workgroup's number mod 8; each in a 128-byte line of its own: arrivals at one address are taken one
// after the other, about 15 ns each, and are 32 this way, not 256); the last arrival of a die counts
// once at the top, and the last of those publishes the barrier's number, which everybody polls.  (All
// workgroups polling the eight counters themselves, with arrivals that nobody waits for, is slower at
// 256 workgroups, 4.7 against 4.0 us a phase: the polls queue up in front of the arrivals.)  The
// counters only ever grow (barrier number e is complete when a counter stands at e times its members),
// so nothing is put back and nothing orders a reset against the next arrival.  One such block serves
// one grid size.
//
// No cache is dropped at the barrier: what a phase hands on is read with device-scope loads.  Dropping
// the die's L2 instead (`buffer_inv sc1`) and reading plainly is correct only if every workgroup does
// it for itself, 50 ns each and one after the other per die (1.7 us a barrier).  One workgroup per die
// doing it for the others (which then drop their first-level cache only) made a barrier of 2.1 us and
// the activations arrive in 2.5 us instead of 3.5, but is wrong now and then: the instruction orders
// the loads of the wavefront that issues it, and nothing tells another compute unit when the L2's
// channels have all carried it out.
struct ProgBarrier {
  unsigned die[8][32];
  unsigned top[32];
  unsigned done[32];   // [0] number of the last complete barrier
  unsigned error[32];  // [0] 0, or 1 + the phase after which a workgroup gave up
};

__device__ __forceinline__ unsigned barrier_members(unsigned die) { return (gridDim.x - die + 7) / 8; }

// Barriers completed before this launch, as the workgroup's own die counter tells (it cannot pass the
// next multiple of its members before this workgroup has arrived).
__device__ __forceinline__ unsigned barrier_epoch_at_start(const ProgBarrier* bar) {
  const unsigned die = blockIdx.x % 8;
  return __hip_atomic_load(&bar->die[die][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) / barrier_members(die);
}

// True when every workgroup has arrived (what they wrote through is then in memory; the reader's caches
// may still hold older copies, which is why it reads such data with device-scope loads); false when the program is dead
// (this workgroup or another gave up), in which case the kernel must end.  `epoch` lives in thread 0.
__device__ __forceinline__ bool grid_barrier(ProgBarrier* bar, unsigned& epoch, int* s_dead, int spin_limit, int phase) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's written-through stores have arrived
  __syncthreads();
  if (threadIdx.x == 0) {
    epoch += 1;
    const unsigned die = blockIdx.x % 8, dies = gridDim.x < 8 ? gridDim.x : 8;
    const unsigned arrived = __hip_atomic_fetch_add(&bar->die[die][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (arrived + 1 == barrier_members(die) * epoch) {
      const unsigned up = __hip_atomic_fetch_add(&bar->top[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (up + 1 == dies * epoch) __hip_atomic_store(&bar->done[0], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    int spins = 0;
    bool alive = true;
    while ((int)(__hip_atomic_load(&bar->done[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - epoch) < 0) {
      if (++spins > spin_limit ||
          (spins % 64 == 0 && __hip_atomic_load(&bar->error[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
        alive = false;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (!alive) {
      __hip_atomic_store(&bar->error[0], (unsigned)(phase + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *s_dead = 1;
    }
  }
  __syncthreads();
  return *s_dead == 0;
}

// ---------------------------------------------------------------------------------------- product
// A product phase is cut into items of 16 weight rows (a tile) by one k range.  A workgroup serves one
// k range (workgroup b the range b % splits; with fewer workgroups than ranges, several in turn): it
// reads the activations of that range once, with device-scope loads, into LDS, in the order in which the
// matrix instruction wants its B operand, and its quads then take the range's tiles in turn, streaming
// only weights.  A quad's four wavefronts take the 32-wide k steps of the range in turn and their sums
// are added in wavefront order through LDS, exactly as gemm_skinny_kernel<1, 1, EPI, 4> adds them.
//
// Weights do not depend on what a barrier waits for, so a wavefront always has its next chunk of them
// (up to PROG_S of its k steps, 14 KB a wavefront) on the way: the next tile's while it multiplies the
// current one, and, across the barrier, the first PROG_AHEAD steps of its first tile of the next phase.
// `coming` carries them from one phase to the next.
#define PROG_S 14  // most k steps of a wavefront whose weights are asked for together (a chunk)
#define PROG_AHEAD 4  // steps of its first chunk of the next phase that a wavefront asks for before the barrier

// Where a wavefront's chunk of weights lies: `steps` steps of 32 from k = kb on, 128 apart, of this
// lane's weight row of width K.  The places past `steps` are asked for from the last step's address
// again (a load that is not made would need a branch, and branches between loads make the compiler
// wait for all of them).
struct Chunk {
  const bf16_t* row;
  int kb, K, steps;
};

template <int S, int FROM = 0>
__device__ __forceinline__ void ask_chunk(bf16x8 (&frag)[PROG_S], const Chunk& c) {
  const int lkg = threadIdx.x % 4;
#pragma unroll
  for (int u = FROM; u < S; ++u) {
    const int uu = u < c.steps ? u : (c.steps > 0 ? c.steps - 1 : 0);
    const int k = c.kb + 128 * uu + 8 * lkg;
    frag[u] = *reinterpret_cast<const bf16x8*>(c.row + (k < c.K - 8 ? k : c.K - 8));
  }
}

// Which tiles of which k range quad `quad` of this workgroup takes: tile first, first + stride, ...
struct Share {
  int range, first, stride;
};
__device__ __forceinline__ Share share_of(int splits, int range_turn, int quad) {
  const int G = gridDim.x, b = blockIdx.x;
  Share sh;
  if (G >= splits) {  // the workgroups whose number is `range` mod splits share the range's tiles
    sh.range = b % splits;
    const int rank = b / splits, count = (G - sh.range + splits - 1) / splits;
    sh.first = rank * PROG_QUADS + quad;
    sh.stride = count * PROG_QUADS;
  } else {            // more ranges than workgroups: a workgroup takes whole ranges in turn
    sh.range = b + range_turn * G;
    sh.first = quad;
    sh.stride = PROG_QUADS;
  }
  return sh;
}

// This lane's weight row of a tile (row lane / 4, through the rotation's row order if any).
__device__ __forceinline__ const bf16_t* weight_row(const ProgPhase& ph, int tile) {
  const int lrow = threadIdx.x % PAE_WAVE / 4;
  int n = 16 * tile + lrow;
  if (ph.epilogue == EPI_ROPE) {
    const int per_head = ph.rope.hd / 16;
    n = tile / per_head * ph.rope.hd + rope_feature(tile % per_head, lrow, ph.rope.rot);
  }
  return in_memory(ph.W) + (int64_t)(n < ph.N ? n : ph.N - 1) * ph.K;  // rows past N are loaded from the last row and never stored
}

// k steps of 32 that one wavefront makes in a k range, at most, and whether its chunks are the short kind
__device__ __forceinline__ int steps_of(const ProgPhase& ph) { return (min(ph.k_per_split, ph.K) + 127) / 128; }
__device__ __forceinline__ bool short_chunks(const ProgPhase& ph) { return steps_of(ph) <= 4; }

// Chunk `c` of wavefront `wq` of a quad for `tile` in k range `range`.
__device__ __forceinline__ Chunk chunk_of(const ProgPhase& ph, int tile, int range, int c, int wq) {
  const int S = short_chunks(ph) ? 4 : PROG_S;
  const int k_lo = range * ph.k_per_split, k_hi = min(ph.K, k_lo + ph.k_per_split);
  const int kb = k_lo + 32 * wq + 128 * S * c;
  const int left = kb < k_hi ? (k_hi - kb + 127) / 128 : 0;
  return Chunk{weight_row(ph, tile), kb, ph.K, left < S ? left : S};
}

// The first chunk of this quad's first tile of phase `next`, if it is a product in which the quad has one.
__device__ __forceinline__ bool first_chunk_of(const ProgPhase* next, int quad, int wq, Chunk& c) {
  if (!next || next->type != PROG_PRODUCT) return false;
  const Share then = share_of(next->splits, 0, quad);
  if (then.range >= next->splits || then.first >= (next->N + 15) / 16) return false;
  c = chunk_of(*next, then.first, then.range, 0, wq);
  return true;
}

__device__ __forceinline__ void product_phase(const ProgPhase& ph, const ProgPhase* next, float* quad_lds, bf16x8* a_lds,
                                              int& parity, bf16x8 (&coming)[PROG_S], bool& has_coming, long long* stamps) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE), quad = wave / 4, wq = wave % 4;
  const int M = ph.M, N = ph.N, K = ph.K, splits = ph.splits;
  const int tiles = (N + 15) / 16;
  const int g4 = lane / 16;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;
  const bool brief = short_chunks(ph);  // the same in the whole grid
  const int S = brief ? 4 : PROG_S, chunks_a_tile = (steps_of(ph) + S - 1) / S;
  float* s_scale = quad_lds + 2 * 3 * 4 * PAE_WAVE;  // [16], behind the two sets of partial sums
  const bf16x8 zero = {};
  const int groups = (int)gridDim.x, group = (int)blockIdx.x;
  const int range_turns = groups >= splits ? 1 : (splits - group + groups - 1) / groups;
  // the quad's chunks of a turn are numbered tile by tile; `in_turn` tells whether chunk j exists and where it lies
  auto in_turn = [&](int turn, int j, Chunk& c) -> bool {
    if (turn >= range_turns) return false;
    const Share sh = share_of(splits, turn, quad);
    const int tile = sh.first + j / chunks_a_tile * sh.stride;
    if (tile >= tiles) return false;
    c = chunk_of(ph, tile, sh.range, j % chunks_a_tile, wq);
    return true;
  };
  const Chunk nothing = {in_memory(ph.W), 0, K, 1};  // asked for where a wavefront has nothing to ask for
  // Of the first chunk only PROG_AHEAD steps were asked for before the barrier, as much as arrives while
  // the barrier is crossed and the activations are fetched; the rest is asked for once the activations are
  // there (asked for earlier, the weights that fast workgroups want fill the memory's queues in front of
  // the activations that slow ones still wait for, and a phase is as slow as its slowest workgroup).
  Chunk first_chunk = nothing;
  in_turn(0, 0, first_chunk);
  bool rest_to_ask = true;
  for (int turn = 0; turn < range_turns; ++turn) {
    const Share sh = share_of(splits, turn, quad);
    const int k_lo = sh.range * ph.k_per_split, k_hi = min(K, k_lo + ph.k_per_split);
    // the range's activations: chunk c of row m (8 elements at k_lo + 8 c) is what lane 16 (c % 4) + m of
    // k step c / 4 multiplies; the last step's chunks past the range are zero (their weights are zeroed
    // too, but zero times whatever LDS held is not always zero)
    const int chunks = (k_hi - k_lo) / 8, padded = (chunks + 3) / 4 * 4;
    if (turn > 0) __syncthreads();  // the range before has been read
    const bf16_t* A = in_memory(ph.A);
    constexpr int AT_ONCE = 4;
    for (int base = threadIdx.x; base < M * padded; base += AT_ONCE * PROG_THREADS) {
      bf16x8 v[AT_ONCE];
#pragma unroll
      for (int q = 0; q < AT_ONCE; ++q) {
        const int idx = base + q * PROG_THREADS, m = idx / padded, c = idx % padded;
        v[q] = zero;
        if (idx < M * padded && c < chunks) v[q] = load_through(reinterpret_cast<const bf16x8*>(A + (int64_t)m * ph.lda + k_lo + 8 * c));
      }
#pragma unroll
      for (int q = 0; q < AT_ONCE; ++q) {
        const int idx = base + q * PROG_THREADS, m = idx / padded, c = idx % padded;
        if (idx < M * padded) a_lds[(c / 4) * PAE_WAVE + (c % 4) * 16 + m] = v[q];
      }
    }
    __syncthreads();
    if (stamps && threadIdx.x == 0 && turn == 0) stamps[2] = wall_clock64();
    if (rest_to_ask) {  // the same in the whole workgroup
      rest_to_ask = false;
      if (!has_coming) {
        if (brief) ask_chunk<4>(coming, first_chunk);
        else ask_chunk<PROG_S>(coming, first_chunk);
      } else if (!brief) {
        ask_chunk<PROG_S, PROG_AHEAD>(coming, first_chunk);
      }
      // what the folded norm owes the rows: the quad's threads together, into the quad's LDS (read after the
      // barrier that follows the first tile's products)
      row_scales_to_lds<1, true, 4>(s_scale, in_memory(ph.norm), M, K, threadIdx.x % (4 * PAE_WAVE), [] {});
    }
    const int rounds = (tiles + sh.stride - 1) / sh.stride;  // the same for the quads of a workgroup
    const int total = rounds * chunks_a_tile;
    f32x4 acc[1][1] = {{(f32x4){0.f, 0.f, 0.f, 0.f}}};
    EpilogueAhead<1> pre = {};
    for (int j = 0; j < total; ++j) {
      bf16x8 cur[PROG_S];
#pragma unroll
      for (int u = 0; u < PROG_S; ++u) cur[u] = coming[u];
      // the chunk after this one, of this range or the next
      if (j + 1 < total || turn + 1 < range_turns) {
        Chunk c = nothing;
        if (j + 1 < total) in_turn(turn, j + 1, c);
        else in_turn(turn + 1, 0, c);
        if (brief) ask_chunk<4>(coming, c);
        else ask_chunk<PROG_S>(coming, c);
      }
      const int tile = sh.first + j / chunks_a_tile * sh.stride, c_in_tile = j % chunks_a_tile;
      const bool live = tile < tiles;  // the same in every lane of the quad
      if (c_in_tile == 0) {
        acc[0][0] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // what the tile's epilogue reads beside the sums is asked for now (by the wavefront that runs it)
        if (live && wq == 0) {
          if (ph.epilogue == EPI_ROPE) ask_row<1, EPI_ROPE>(pre, M, in_memory(ph.rope));
          if (ph.epilogue == EPI_ROPE) ask_epilogue<1, EPI_ROPE, false>(pre, tile, nullptr, 0, M, N, in_memory(ph.rope), SkinnyNorm{});
          if (ph.epilogue == EPI_RESIDUAL) ask_epilogue<1, EPI_RESIDUAL, true>(pre, tile, in_memory(ph.out), ph.ldc, M, N, SkinnyRope{}, in_memory(ph.norm));
        }
      }
      if (live) {
        const int kb = k_lo + 32 * wq + 128 * S * c_in_tile;
        auto multiply = [&](auto steps) {
#pragma unroll
          for (int u = 0; u < decltype(steps)::value; ++u) {
            // four steps' operands at a time (read ahead for a whole chunk they would not fit the registers)
            if (u % 4 == 0 && u > 0) asm volatile("" ::: "memory");
            const int k = kb + 128 * u;  // this wavefront's step: k .. k + 31
            const bool kok = k + 8 * g4 < k_hi;
            // (past the range the step's place in LDS is the last one's: its weights are zero)
            const bf16x8 a = a_lds[(min(k, k_hi - 1) - k_lo) / 32 * PAE_WAVE + lane];
            const bf16x8 moved = to_mfma_order(cur[u], fetch_from);
            acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kok ? moved : zero, a, acc[0][0], 0, 0, 0);
          }
        };
        if (brief) multiply(std::integral_constant<int, 4>{});
        else multiply(std::integral_constant<int, PROG_S>{});
      }
      if (stamps && threadIdx.x == 0 && turn == 0 && j == 0) stamps[3] = wall_clock64();
      if (c_in_tile + 1 < chunks_a_tile) continue;
      // the tile's sums: the four wavefronts' in wavefront order, then the k ranges', then the epilogue
      float* s_part = quad_lds + parity * (3 * 4 * PAE_WAVE);  // [3][4][64]
      parity ^= 1;
      if (live && wq > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s_part[((wq - 1) * 4 + i) * PAE_WAVE + lane] = acc[0][0][i];
      }
      __syncthreads();
      if (stamps && threadIdx.x == 0 && turn == 0 && j + 1 == chunks_a_tile) stamps[4] = wall_clock64();
      if (!live || wq > 0) continue;
#pragma unroll
      for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[0][0][i] += s_part[(w * 4 + i) * PAE_WAVE + lane];
      const float scale[1] = {s_scale[lane % 16]};
      if (ph.epilogue != EPI_F32 && splits > 1) {
        f32x4 mine[1] = {acc[0][0]};
        if (!add_up_k_ranges<1, 4>(mine, tile, sh.range, splits, SkinnyTickets{in_memory(ph.ticket_parts), in_memory(ph.ticket_counters)})) continue;
        acc[0][0] = mine[0];
      }
#define PROG_EPILOGUE(EPI)                                                                                          \
  skinny_epilogue<1, 1, EPI, true>(acc, tile, -1, in_memory(ph.out), ph.ldc, in_memory(ph.bias), ph.b_is_f32, M, N, sh.range, \
                                   (int64_t)M * N, in_memory(ph.rope), in_memory(ph.norm), scale, AHEAD)
      switch (ph.epilogue) {  // the one place where the epilogues part ways: the products above are the same code for all
#define AHEAD nullptr
        case EPI_BF16: PROG_EPILOGUE(EPI_BF16); break;
        case EPI_F32: PROG_EPILOGUE(EPI_F32); break;
        case EPI_SWIGLU: PROG_EPILOGUE(EPI_SWIGLU); break;
#undef AHEAD
#define AHEAD &pre
        case EPI_ROPE: PROG_EPILOGUE(EPI_ROPE); break;
        default: PROG_EPILOGUE(EPI_RESIDUAL); break;
#undef AHEAD
      }
#undef PROG_EPILOGUE
      if (stamps && threadIdx.x == 0 && turn == 0 && j + 1 == chunks_a_tile) stamps[5] = wall_clock64();
    }
  }
  // the weights of this quad's first tile of the next phase, on their way while the barrier is crossed
  Chunk then;
  has_coming = first_chunk_of(next, quad, wq, then);
  if (has_coming) ask_chunk<PROG_AHEAD>(coming, then);
}

// -------------------------------------------------------------------------------------- attention
// Item i is split i % max_splits of key/value head (i / max_splits) % nkv of token i / (max_splits *
// nkv); items whose split lies outside the token's keys are empty.  Inside an item the quad is
// attn_decode_kernel's workgroup; it leaves its partial result in memory for the merge phase.
//
// The queries, the page that holds the token's own key and value (written by the phase before) and
// the partial results are read with device-scope loads; every other page has not been written since
// the kernel began and is read plainly.
template <int HD>
__device__ __forceinline__ void load_kv_tile_through(bf16x8 (&kf)[HD / 32], s16x4 (&vf)[HD / 16], const bf16_t* kp,
                                                     const bf16_t* vp, int vstride) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int r = lane / 4, g = lane % 4;
#pragma unroll
  for (int j = 0; j < HD / 32; ++j) kf[j] = load_through(reinterpret_cast<const bf16x8*>(kp + r * HD + 32 * j + 8 * g));
#pragma unroll
  for (int t = 0; t < HD / 16; ++t)
    vf[t] = load_through(reinterpret_cast<const s16x4*>(vp + (int64_t)(16 * t + lane % 16) * vstride + 4 * (lane / 16)));
}

template <int HD>
__device__ __forceinline__ void attention_phase(const ProgPhase& ph, float* quad_lds, long long* stamps) {
  constexpr int TPW = PROG_SPLIT / 64, ROWS = HD / 4 + 2;
  const int lane = threadIdx.x % PAE_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE), quad = wave / 4, wq = wave % 4;
  const int col = lane % 16, g4 = lane / 16;
  const int nkv = ph.nkv, g = ph.nh / nkv, bs = ph.bs, window = ph.window, max_splits = ph.max_splits;
  const int items = ph.num_dec * nkv * max_splits, per_round = gridDim.x * PROG_QUADS;
  const int page_elems = bs * HD;
  for (int base = 0; base < items; base += per_round) {
    const int item = base + quad * gridDim.x + blockIdx.x;
    bool live = item < items;
    const int split = live ? item % max_splits : 0, kvh = live ? item / max_splits % nkv : 0;
    const int tok_index = live ? item / (max_splits * nkv) : 0;
    const int4 work = in_memory(ph.dec_work)[tok_index];
    const int pos[1] = {work.y};
    const int start[1] = {(window > 0 && pos[0] - window + 1 > 0) ? pos[0] - window + 1 : 0};
    const int s_first = start[0] / PROG_SPLIT, s_last = pos[0] / PROG_SPLIT;
    live = live && split >= s_first && split <= s_last;
    AttnState<HD, 1> st;
    st.m[0] = NEG_BIG;
    st.l[0] = 0.f;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) st.acc[0][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (live) {
      const int lo = max(split * PROG_SPLIT, start[0] / 16 * 16);
      const int hi = min((split + 1) * PROG_SPLIT, pos[0] + 1);
      const int* table = in_memory(ph.block_tables) + (int64_t)work.z * ph.max_blocks;
      const int tile_lo = lo / 16, tile_hi = (hi + 15) / 16, own_tile = pos[0] / 16;
      bf16x8 kf[TPW][HD / 32];
      s16x4 vf[TPW][HD / 16];
#pragma unroll
      for (int j = 0; j < TPW; ++j) {  // a tile past the end is loaded from the first tile's place and not used
        const int tile = tile_lo + wq + 4 * j;
        const int key0 = (tile < tile_hi ? tile : tile_lo) * 16;
        const int64_t at = ((int64_t)table[key0 / bs] * nkv + kvh) * page_elems;
        const bf16_t* kp = in_memory(ph.k_cache) + at + (int64_t)(key0 % bs) * HD;
        const bf16_t* vp = in_memory(ph.v_cache) + at + key0 % bs;
        if (key0 / 16 == own_tile) load_kv_tile_through<HD>(kf[j], vf[j], kp, vp, bs);  // the same in the whole wavefront
        else load_kv_tile<HD>(kf[j], vf[j], kp, vp, bs);
      }
      bf16x8 qf[1][HD / 32];
      const bf16_t* qrow = in_memory(ph.q) + (int64_t)work.x * ph.q_stride + (int64_t)(kvh * g + (col < g ? col : 0)) * HD;
#pragma unroll
      for (int j = 0; j < HD / 32; ++j) {
        qf[0][j] = load_through(reinterpret_cast<const bf16x8*>(qrow + 32 * j + 8 * g4));
        if (col >= g)
#pragma unroll
          for (int e = 0; e < 8; ++e) qf[0][j][e] = (__bf16)0.f;
      }
#pragma unroll
      for (int j = 0; j < TPW; ++j) {
        const int tile = tile_lo + wq + 4 * j;
        keys_to_mfma_order<HD>(kf[j]);
        if (tile < tile_hi) attn_tile<HD, 1>(st, kf[j], vf[j], qf, tile * 16, pos, start, ph.scale_log2);
      }
      if (stamps && threadIdx.x == 0 && base == 0) stamps[2] = wall_clock64();
      if (wq > 0) {
        float* mine = quad_lds + (wq - 1) * ROWS * PAE_WAVE;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[(4 * t + i) * PAE_WAVE + lane] = st.acc[0][t][i];
        mine[(HD / 4) * PAE_WAVE + lane] = st.m[0];
        mine[(HD / 4 + 1) * PAE_WAVE + lane] = st.l[0];
      }
    }
    __syncthreads();
    if (live && wq == 0) {
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        const float* theirs = quad_lds + w * ROWS * PAE_WAVE;
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
      const int pair = tok_index * nkv + kvh;
      if (col < g) {
        const int64_t slot = ((int64_t)pair * max_splits + split) * g + col;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t)
          put<true>(reinterpret_cast<f32x4*>(in_memory(ph.part_acc) + slot * HD + 16 * t + 4 * g4), st.acc[0][t]);
        if (g4 == 0) {
          put<true>(in_memory(ph.part_ml) + slot * 2, st.m[0]);
          put<true>(in_memory(ph.part_ml) + slot * 2 + 1, l);
        }
      }
    }
    if (stamps && threadIdx.x == 0 && base == 0) stamps[3] = wall_clock64();
    __syncthreads();  // the quads' LDS is free for the next round
  }
}

// The merge of a (token, key/value head)'s splits, after the barrier that follows the attention
// phase.  Item i is 64 of the (head of the group, four features) of pair i / per_pair; the quad's four
// wavefronts are attn_decode_merge_kernel's four groups of splits (wavefront w adds the splits first +
// w, + 4, ... in split order), and wavefront 0 then adds the groups' sums in group order.
#define PROG_MERGE_BATCH 12  // splits of one wavefront whose partial results are in flight together

template <int HD>
__device__ __forceinline__ void merge_phase(const ProgPhase& ph, float* quad_lds) {
  const int lane = threadIdx.x % PAE_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PAE_WAVE), quad = wave / 4, wq = wave % 4;
  const int nkv = ph.nkv, g = ph.nh / nkv, window = ph.window, max_splits = ph.max_splits;
  const int merge_items = g * (HD / 4), per_pair = (merge_items + PAE_WAVE - 1) / PAE_WAVE;
  const int items = ph.num_dec * nkv * per_pair, per_round = gridDim.x * PROG_QUADS;
  for (int base = 0; base < items; base += per_round) {
    const int item = base + quad * gridDim.x + blockIdx.x;
    const bool live = item < items;
    const int pair = live ? item / per_pair : 0;
    const int it = (live ? item % per_pair : 0) * PAE_WAVE + lane;
    const bool mine = live && it < merge_items;
    const int c = mine ? it / (HD / 4) : 0, d = (it % (HD / 4)) * 4;
    const int4 mw = in_memory(ph.dec_work)[pair / nkv];
    const int m_tok = mw.x, m_kvh = pair % nkv;
    const int mstart = (window > 0 && mw.y - window + 1 > 0) ? mw.y - window + 1 : 0;
    const int m_first = mstart / PROG_SPLIT, m_count = mw.y / PROG_SPLIT - m_first + 1;
    float m = NEG_BIG, l = 0.f;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    if (live) {
      const int64_t slot0 = ((int64_t)pair * max_splits + m_first) * g + c;
      for (int sp0 = wq; sp0 < m_count; sp0 += 4 * PROG_MERGE_BATCH) {
        f32x4 v[PROG_MERGE_BATCH];
        float ms[PROG_MERGE_BATCH], ls[PROG_MERGE_BATCH];
#pragma unroll
        for (int j = 0; j < PROG_MERGE_BATCH; ++j) {
          const int sp = sp0 + 4 * j;
          const int64_t slot = slot0 + (int64_t)(sp < m_count ? sp : sp0) * g;  // past the end: the batch's first, not used
          v[j] = load_through(reinterpret_cast<const f32x4*>(in_memory(ph.part_acc) + slot * HD + d));
          const unsigned long long raw = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(in_memory(ph.part_ml) + slot * 2),
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ms[j] = __uint_as_float((unsigned)raw);
          ls[j] = __uint_as_float((unsigned)(raw >> 32));
        }
#pragma unroll
        for (int j = 0; j < PROG_MERGE_BATCH; ++j) {
          if (sp0 + 4 * j >= m_count) break;
          const float m_new = fmaxf(m, ms[j]);
          const float f_old = exp2f(m - m_new), f = exp2f(ms[j] - m_new);
          a = a * f_old + v[j] * f;
          l = l * f_old + ls[j] * f;
          m = m_new;
        }
      }
      if (wq > 0) {
        float* dst = quad_lds + ((int64_t)(wq - 1) * PAE_WAVE + lane) * 6;
        dst[0] = a[0]; dst[1] = a[1]; dst[2] = a[2]; dst[3] = a[3]; dst[4] = m; dst[5] = l;
      }
    }
    __syncthreads();
    if (mine && wq == 0) {
      for (int other = 1; other < 4; ++other) {
        const float* src = quad_lds + ((int64_t)(other - 1) * PAE_WAVE + lane) * 6;
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
      put<true>(reinterpret_cast<s16x4*>(in_memory(ph.attn_out) + (int64_t)m_tok * ph.out_stride + (int64_t)(m_kvh * g + c) * HD + d), w);
    }
    __syncthreads();  // the quads' LDS is free for the next round
  }
}

__global__ __launch_bounds__(PROG_THREADS) void decode_program_kernel(const ProgPhase* phases, int num_phases,
                                                                      ProgBarrier* bar, int* host_error,
                                                                      int quad_floats, int spin_limit,
                                                                      long long* trace) {
  // dynamic LDS: the quads' regions (sums of a quad's wavefronts, attention states, merges), then the
  // region for a product's activations
  extern __shared__ float s_mem[];
  __shared__ int s_dead;
  // The phase's description lives in LDS while the phase runs (read from memory, every use of a field
  // after a store or a fence would be a trip of its own), and the next phase's is fetched before the
  // barrier, so that its trip is over when the barrier opens.
  __shared__ __align__(16) ProgPhase s_phase[3];
  constexpr int PIECES = (int)(sizeof(ProgPhase) / 16);
  int4 piece = {};  // this thread's 16 bytes of a coming phase's description, on their way
  auto ask_for_phase = [&](int p) {
    if (threadIdx.x < PIECES) piece = reinterpret_cast<const int4*>(phases + p)[threadIdx.x];
  };
  auto keep_phase = [&](int p) {
    if (threadIdx.x < PIECES) reinterpret_cast<int4*>(&s_phase[p % 3])[threadIdx.x] = piece;
  };
  float* quad_lds = s_mem + (int64_t)(threadIdx.x / (4 * PAE_WAVE)) * quad_floats;
  bf16x8* a_lds = reinterpret_cast<bf16x8*>(s_mem + (int64_t)PROG_QUADS * quad_floats);
  unsigned epoch = 0;
  if (threadIdx.x == 0) {
    s_dead = 0;
    epoch = barrier_epoch_at_start(bar);
  }
  // phase p runs from s_phase[p % 3]; the description of phase p + 1 is there as well (a quad asks for
  // its first weights of the next phase before the barrier), and that of phase p + 2 is on its way
  ask_for_phase(0);
  keep_phase(0);
  if (num_phases > 1) {
    ask_for_phase(1);
    keep_phase(1);
  }
  __syncthreads();
  int parity = 0;
  bf16x8 coming[PROG_S] = {};  // a wavefront's next chunk of weights, asked for ahead (see product_phase)
  bool has_coming = false;
  for (int p = 0; p < num_phases; ++p) {
    const ProgPhase& ph = s_phase[p % 3];
    const ProgPhase* next = p + 1 < num_phases ? &s_phase[(p + 1) % 3] : nullptr;
    if (p + 2 < num_phases) ask_for_phase(p + 2);  // kept when this phase is over
    if (trace && threadIdx.x == 0) {
      trace[((int64_t)p * gridDim.x + blockIdx.x) * PROG_STAMPS] = wall_clock64();
      trace[((int64_t)p * gridDim.x + blockIdx.x) * PROG_STAMPS + 7] = __builtin_amdgcn_s_getreg((3 << 11) | 20);  // XCC_ID
    }
    long long* stamps = trace ? trace + ((int64_t)p * gridDim.x + blockIdx.x) * PROG_STAMPS : nullptr;
    if (ph.type == PROG_PRODUCT) {
      product_phase(ph, next, quad_lds, a_lds, parity, coming, has_coming, stamps);
    } else {
      if (ph.type == PROG_ATTENTION) {
        if (ph.hd == 128) attention_phase<128>(ph, quad_lds, stamps);
        else attention_phase<64>(ph, quad_lds, stamps);
      } else {
        if (ph.hd == 128) merge_phase<128>(ph, quad_lds);
        else merge_phase<64>(ph, quad_lds);
      }
      has_coming = false;  // nothing is carried across an attention phase: the registers are free during it
#pragma unroll
      for (int u = 0; u < PROG_S; ++u) coming[u] = bf16x8{};
    }
    if (trace && threadIdx.x == 0) trace[((int64_t)p * gridDim.x + blockIdx.x) * PROG_STAMPS + 1] = wall_clock64();
    if (p + 1 == num_phases) break;
    // into the buffer of phase p - 1, whose last readers passed the barrier's workgroup barriers a phase ago
    if (p + 2 < num_phases) keep_phase(p + 2);
    if (!grid_barrier(bar, epoch, &s_dead, spin_limit, p)) {
      if (threadIdx.x == 0 && blockIdx.x == 0) *host_error = p + 1;
      return;
    }
  }
}

// ---------------------------------------------------------------------------------- host side
extern "C" int pae_program_phase_bytes() { return (int)sizeof(ProgPhase); }
extern "C" int pae_program_barrier_bytes() { return (int)sizeof(ProgBarrier); }
extern "C" int pae_program_max_rows() { return PROG_MAX_ROWS; }

static int quad_bytes_of_product() { return (2 * 3 * 4 * PAE_WAVE + 16) * (int)sizeof(float); }

// Bytes of LDS that the activations of one k range of a product take in a workgroup: `rows` rows of one
// range, whole k steps of 32.
extern "C" int pae_program_activation_bytes(int rows, int K, int splits) {
  if (rows < 1 || K < 1 || splits < 1) return 0;
  int k_per_split = (K + splits - 1) / splits;
  k_per_split = (k_per_split + 127) / 128 * 128;
  if (k_per_split > K) k_per_split = (K + 31) / 32 * 32;
  return k_per_split / 32 * PAE_WAVE * 16;
}
extern "C" int pae_program_lds_limit();

// Writes phase `index` of the host-side list `phases`: a product with any epilogue but the rotating
// one.  Arguments as pae_gemm_skinny; the k ranges are those that call would take.  Returns the
// bytes of LDS a quad needs for the phase, or a negative code.
extern "C" int pae_program_put_product(void* phases, int index, int epilogue, void* out, int64_t ldc, const void* A,
                                       int64_t lda, const void* W, const void* bias, int b_is_f32, int M, int N, int K,
                                       int splits, float* ticket_parts, int* ticket_counters, const float* row_stats,
                                       int row_stat_tiles, float row_eps, void* next_rows, int64_t ld_next,
                                       const void* next_w, int next_w_is_f32, float* next_stats, const SkinnyRope* rope) {
  PAE_REQUIRE(phases && index >= 0, "decode program: no room for phase %d", index);
  PAE_REQUIRE(M >= 1 && M <= PROG_MAX_ROWS, "decode program: a product of %d rows (1..%d are taken)", M, PROG_MAX_ROWS);
  PAE_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && lda % 8 == 0, "decode program: N=%d K=%d lda=%lld (K and lda must be multiples of 8)",
              N, K, (long long)lda);
  PAE_REQUIRE(epilogue == EPI_BF16 || epilogue == EPI_F32 || epilogue == EPI_SWIGLU || epilogue == EPI_RESIDUAL ||
              (epilogue == EPI_ROPE && rope), "decode program: unknown epilogue %d", epilogue);
  const bool ticketed = splits > 1 && epilogue != EPI_F32;
  PAE_REQUIRE(splits >= 1 && (!ticketed || (ticket_parts && ticket_counters)),
              "decode program: %d k ranges with epilogue %d need scratch for partial sums and tickets", splits, epilogue);
  PAE_REQUIRE(!(bias && splits > 1 && !ticketed), "decode program: a bias cannot be combined with partial sums");
  PAE_REQUIRE(!row_stats || row_stat_tiles > 0, "decode program: a row scale needs its shares of the sums of squares");
  PAE_REQUIRE(epilogue != EPI_RESIDUAL || (next_rows && next_w && next_stats && ld_next >= N && !bias),
              "decode program: the residual epilogue needs the next rows, the next norm's weight and room for its sums, and takes no bias");
  PAE_REQUIRE(epilogue != EPI_SWIGLU || (N % 16 == 0 && ldc % 4 == 0), "decode program: gated epilogue needs N %% 16 == 0, got %d", N);
  PAE_REQUIRE(epilogue != EPI_ROPE || N % 16 == 0, "decode program: the rotating epilogue needs whole tiles, N=%d", N);
  int k_per_split = (K + splits - 1) / splits;
  k_per_split = (k_per_split + 127) / 128 * 128;
  PAE_REQUIRE((int64_t)k_per_split * (splits - 1) < K, "decode program: %d k ranges are too many for K=%d", splits, K);
  ProgPhase ph = {};
  ph.type = PROG_PRODUCT;
  ph.epilogue = epilogue;
  ph.M = M; ph.N = N; ph.K = K; ph.splits = splits; ph.k_per_split = k_per_split; ph.b_is_f32 = b_is_f32;
  ph.W = (const bf16_t*)W; ph.bias = bias; ph.A = (const bf16_t*)A; ph.out = out;
  ph.lda = lda; ph.ldc = ldc;
  ph.norm = SkinnyNorm{row_stats, row_stat_tiles, row_eps, (bf16_t*)next_rows, ld_next, next_w, next_w_is_f32, next_stats};
  if (rope) ph.rope = *rope;
  ph.ticket_parts = ticketed ? ticket_parts : nullptr;
  ph.ticket_counters = ticketed ? ticket_counters : nullptr;
  ((ProgPhase*)phases)[index] = ph;
  return quad_bytes_of_product();
}

// The query/key/value product with rotation and cache write; arguments as pae_gemm_skinny_rope.
extern "C" int pae_program_put_product_rope(void* phases, int index, void* q_out, int64_t ldq, const void* A, int64_t lda,
                                            const void* W, const void* bias, int b_is_f32, int M, int K, int nh, int nkv,
                                            int hd, int rot, const float* cos_sin, const int* positions,
                                            const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                                            void* k_cache, void* v_cache, int splits, float* ticket_parts,
                                            int* ticket_counters, const float* row_stats, int row_stat_tiles,
                                            float row_eps) {
  PAE_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && hd % 16 == 0, "decode program: bad head sizes nh=%d nkv=%d hd=%d", nh, nkv, hd);
  PAE_REQUIRE(rot >= 0 && rot <= hd && rot % 16 == 0 && (rot == 0 || cos_sin),
              "decode program: rotary_dim %d must be a multiple of 16 up to head_dim %d", rot, hd);
  PAE_REQUIRE(ldq >= (int64_t)nh * hd && ldq % 4 == 0, "decode program: row stride %lld of the queries", (long long)ldq);
  PAE_REQUIRE(positions, "decode program: positions are missing");
  PAE_REQUIRE(nkv == 0 || (bs > 0 && max_blocks > 0 && k_cache && v_cache && block_tables && tok_seq),
              "decode program: the cache write needs tables and pools");
  const SkinnyRope rope{cos_sin, positions, tok_seq, block_tables, (bf16_t*)k_cache, (bf16_t*)v_cache,
                        nh, nkv, hd, rot, max_blocks, bs};
  return pae_program_put_product(phases, index, EPI_ROPE, q_out, ldq, A, lda, W, bias, b_is_f32, M, (nh + 2 * nkv) * hd, K,
                                 splits, ticket_parts, ticket_counters, row_stats, row_stat_tiles, row_eps, nullptr, 0,
                                 nullptr, 0, nullptr, &rope);
}

// Decode attention of num_dec tokens; arguments as pae_attn_decode_bf16.  Writes two phases, index and
// index + 1: the splits' partial results, and their merge.
extern "C" int pae_program_put_attention(void* phases, int index, void* out, int64_t out_stride, const void* q,
                                         int64_t q_stride, const void* k_cache, const void* v_cache, const int* dec_work,
                                         int num_dec, const int* block_tables, int max_blocks, int bs, int nh, int nkv,
                                         int hd, float scale, int window, void* part_acc, void* part_ml) {
  PAE_REQUIRE(phases && index >= 0, "decode program: no room for phase %d", index);
  PAE_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0 && nh / nkv <= 16, "decode program: %d query heads over %d key/value heads", nh, nkv);
  PAE_REQUIRE(hd == 64 || hd == 128, "decode program: attention takes head_dim 64 or 128, got %d", hd);
  PAE_REQUIRE(bs >= 16 && bs % 16 == 0 && max_blocks > 0 && window >= 0, "decode program: page size %d, table width %d, window %d",
              bs, max_blocks, window);
  PAE_REQUIRE(num_dec >= 1 && num_dec <= PROG_MAX_ROWS && dec_work && block_tables && part_acc && part_ml,
              "decode program: attention of %d tokens (1..%d are taken) needs its work list, tables and scratch",
              num_dec, PROG_MAX_ROWS);
  ProgPhase ph = {};
  ph.type = PROG_ATTENTION;
  ph.dec_work = (const int4*)dec_work; ph.block_tables = block_tables;
  ph.q = (const bf16_t*)q; ph.attn_out = (bf16_t*)out;
  ph.k_cache = (const bf16_t*)k_cache; ph.v_cache = (const bf16_t*)v_cache;
  ph.part_acc = (float*)part_acc; ph.part_ml = (float*)part_ml;
  ph.q_stride = q_stride; ph.out_stride = out_stride;
  ph.num_dec = num_dec;
  ph.max_splits = (int)(((int64_t)max_blocks * bs + PROG_SPLIT - 1) / PROG_SPLIT);
  ph.max_blocks = max_blocks; ph.bs = bs; ph.nh = nh; ph.nkv = nkv; ph.hd = hd; ph.window = window;
  ph.scale_log2 = scale * LOG2E;
  ((ProgPhase*)phases)[index] = ph;
  ph.type = PROG_MERGE;
  ((ProgPhase*)phases)[index + 1] = ph;
  const int state = 3 * (hd / 4 + 2) * PAE_WAVE, merge = 3 * PAE_WAVE * 6;
  return (state > merge ? state : merge) * (int)sizeof(float);
}

// The most workgroups that can be resident at once on the current device (one per compute unit: the
// kernel takes all of a unit's registers); also asks the runtime for the kernel's LDS.  Call it once per device before
// the first pae_program_run there, outside any stream capture.
#define PROG_LDS_LIMIT (160 * 1024 - 2048)  // dynamic LDS: what the kernel declares for itself (phase descriptions, flags) stays below 2 KB
static int g_max_groups[64];

extern "C" int pae_program_lds_limit() { return PROG_LDS_LIMIT; }

extern "C" int pae_program_max_groups() {
  int dev = 0, units = 0, per_unit = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess || dev < 0 || dev >= 64) return pae_fail("decode program: no usable current device");
  if (g_max_groups[dev] > 0) return g_max_groups[dev];
  err = hipFuncSetAttribute((const void*)decode_program_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, PROG_LDS_LIMIT);
  if (err != hipSuccess) return pae_fail("decode program: cannot ask for LDS: %s", hipGetErrorString(err));
  err = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev);
  if (err == hipSuccess)
    err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, (const void*)decode_program_kernel, PROG_THREADS,
                                                       PROG_LDS_LIMIT);
  if (err != hipSuccess) return pae_fail("decode program: cannot tell how many workgroups fit: %s", hipGetErrorString(err));
  PAE_REQUIRE(units * per_unit >= 1, "decode program: the kernel does not fit a compute unit");
  g_max_groups[dev] = units * per_unit;
  return g_max_groups[dev];
}

// Runs phases[0 .. num_phases) (device memory) on `groups` resident workgroups.  `barrier` is
// pae_program_barrier_bytes() of device memory, zero before its first use and used with one value of
// `groups` only; `host_error` is an int in pinned host memory that receives 1 + the phase at whose
// barrier a workgroup gave up after `spin_limit` polls (it stays as it is otherwise).  Launches that
// share a barrier block or ticket counters must not overlap.  `trace` (or null): device memory for
// num_phases * groups * 8 numbers: clock readings (100 MHz) [0] when the workgroup began the phase, [1] when it
// ended it, [2..5] marks of the phase's own (product: activations in LDS, first chunk multiplied, first tile's
// sums added, its epilogue done; attention: first item computed, its partial result stored), and [7] the number
// of the die that the workgroup ran on (the barrier counts on it being the workgroup's number mod 8).
extern "C" int pae_program_run(const void* phases, int num_phases, void* barrier, int* host_error, int groups,
                               int quad_lds_bytes, int activation_lds_bytes, int spin_limit, long long* trace,
                               hipStream_t stream) {
  PAE_REQUIRE(phases && barrier && host_error && num_phases >= 1, "decode program: nothing to run");
  PAE_REQUIRE(quad_lds_bytes >= quad_bytes_of_product() && quad_lds_bytes % 16 == 0 && activation_lds_bytes >= 0 &&
              activation_lds_bytes % 16 == 0 && (int64_t)quad_lds_bytes * PROG_QUADS + activation_lds_bytes <= PROG_LDS_LIMIT,
              "decode program: %d bytes of LDS a quad and %d for a product's activations exceed the %d there are",
              quad_lds_bytes, activation_lds_bytes, PROG_LDS_LIMIT);
  PAE_REQUIRE(spin_limit > 0, "decode program: the waits must be bounded");
  int dev = 0;
  PAE_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && g_max_groups[dev] > 0,
              "decode program: pae_program_max_groups has not been called on this device");
  // every workgroup must be resident at once, or the barrier between the phases never completes
  PAE_REQUIRE(groups >= 1 && groups <= g_max_groups[dev], "decode program: %d workgroups cannot all be resident (at most %d)",
              groups, g_max_groups[dev]);
  decode_program_kernel<<<groups, PROG_THREADS, (size_t)quad_lds_bytes * PROG_QUADS + activation_lds_bytes, stream>>>(
      (const ProgPhase*)phases, num_phases, (ProgBarrier*)barrier, host_error, quad_lds_bytes / (int)sizeof(float), spin_limit,
      trace);
  return pae_check_launch("decode program");
}
