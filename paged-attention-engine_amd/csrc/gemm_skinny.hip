// C[M,N] = A[M,K] * W[N,K]^T for few rows (M <= 64): the matrix products of a
// decode step, which are bound by reading W once from HBM.
//
// W (bfloat16, (out_features, in_features) row-major as in the checkpoint) is the
// A operand of MFMA 16x16x32, 16 weight rows per tile; the activations are the B
// operand, 16 rows of A per column tile, so each weight fragment is loaded once
// and used for every row of A.  A workgroup owns 16 weight rows (32 for the gated
// epilogue) and a range of k; its four wavefronts take 32-wide k steps in turn
// and are summed in LDS in wavefront order.  With several k ranges (grid.y > 1)
// each writes its own float32 partial, which the consumer adds up in range
// order: no atomics, the same sums in the same order on every run.
//
// Epilogues: bfloat16 out with bias; float32 out (logits, or partial sums);
// SiLU gate: rows come in blocks of 8 gate rows followed by their 8 up rows (one tile of the
// matrix instruction holds both), and out[m, j] = silu(gate_j) * up_j (engine/model.py:317-320 of the reference);
// rotation: W holds the query, key and value projections of an attention layer, a
// tile takes 8 features of a head and the 8 they are rotated with, queries come out
// rotated and keys and values go straight to their cache slots (engine/model.py:
// 155-161, engine/attention.py:374-385,409-410), so the projection's result never
// makes a round trip through memory.
#include "common.h"
#include "api.h"
#include "skinny_device.h"

// MT: column tiles of 16 rows of A; RT: tiles of 16 weight rows per workgroup; SKINNY_U: k steps
// of a wavefront whose loads are in flight together.  With more
// rows of A a workgroup takes more weight rows, so that the activations, which every
// workgroup re-reads from L2, do not outweigh the weights.
template <int MT, int RT, int EPI, int SKINNY_U, int NW = 4>
__global__ __launch_bounds__(64 * NW) void gemm_skinny_kernel(void* __restrict__ out, int64_t ldc,
                                                          const bf16_t* __restrict__ A, int64_t lda,
                                                          const bf16_t* __restrict__ W,
                                                          const void* __restrict__ bias, int b_is_f32, int M,
                                                          int N, int K, int k_per_split, int64_t part_stride,
                                                          SkinnyRope rope, SkinnyTickets tickets, SkinnyNorm norm) {
  // NW == 16 (one column tile only): the workgroup holds four k ranges side by side, four wavefronts to
  // each, and adds the ranges' sums in range order itself: the sums, bit for bit, of four workgroups
  // with one range each whose results the last to finish adds up (grid.y == 4), without the tickets
  // and the trip to memory.
  static_assert(NW == 4 || (NW == 16 && MT == 1), "sixteen wavefronts only with one column tile");
  __shared__ float s_part[MT == 1 ? NW - 1 : 4][RT * MT * 4][PAE_WAVE];
  __shared__ float s_scale[16 * MT];  // what the folded norm owes every row of A
  if (MT == 1 && gridDim.z > 1) {  // the rows of A are shared out in tiles of 16: this workgroup's tile
    const int m0 = blockIdx.z * 16;
    A += (int64_t)m0 * lda;
    out = (EPI == EPI_F32 || EPI == EPI_RESIDUAL) ? (void*)((float*)out + (int64_t)m0 * ldc)
                                                  : (void*)((bf16_t*)out + (int64_t)m0 * ldc);
    M = min(16, M - m0);
    if (norm.row_stats) norm.row_stats += (int64_t)m0 * norm.row_stat_tiles;
    if (EPI == EPI_RESIDUAL) {
      norm.next_rows += (int64_t)m0 * norm.ld_next;
      norm.next_stats += (int64_t)m0 * ((N + 15) / 16);
    }
    if (EPI == EPI_ROPE) {
      rope.positions += m0;
      if (rope.tok_seq) rope.tok_seq += m0;
      if (rope.cos_sin) rope.cos_sin += (int64_t)m0 * rope.rot;
    }
  }
  const int tid = threadIdx.x, lane = tid % PAE_WAVE, wave = tid / PAE_WAVE;
  const int r = lane % 16, g4 = lane / 16;
  // with one column tile, what the epilogue reads is asked for before the products
  constexpr bool AHEAD = MT == 1 && (EPI == EPI_RESIDUAL || EPI == EPI_ROPE);
  EpilogueAhead<RT> ahead;
  const int n0 = blockIdx.x * 16 * RT;
  const int k_lo = (NW == 16 ? wave / 4 : blockIdx.y) * k_per_split;
  const int k_hi = min(K, k_lo + k_per_split);

  // Loads are made with the lane order (row = lane / 4, k group = lane % 4): the four lanes of a
  // quad then read 64 contiguous bytes, which the memory pipeline handles as one access.  The
  // matrix instruction wants (row = lane % 16, k group = lane / 16); one cross-lane permute per
  // register moves a loaded fragment into that order.
  const int lrow = lane / 4, lkg = lane % 4;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;  // byte address of the source lane for ds_bpermute
  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n = n0 + 16 * rt + lrow;
    if (EPI == EPI_ROPE) {
      const int tile = blockIdx.x * RT + rt, per_head = rope.hd / 16;
      n = tile / per_head * rope.hd + rope_feature(tile % per_head, lrow, rope.rot);
    }
    wrow[rt] = W + (int64_t)(n < N ? n : N - 1) * K;  // rows past N are loaded from the last row and never stored
  }
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + lrow;
    arow[mt] = A + (int64_t)(m < M ? m : M - 1) * lda;
  }
  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // Every lane of a wavefront runs the same number of steps (the matrix instruction
  // takes operands from all 64 lanes).  Loads are unconditional, from clamped
  // addresses, and issued SKINNY_U steps ahead of their use; a lane past the end of
  // the k range zeroes its weight fragment (rows past N or M are simply not stored).
  const bf16x8 zero = {};
  constexpr int KW = 128;  // a range's four wavefronts take 32-wide k steps in turn
  struct Batch {  // SKINNY_U steps of a wavefront: k offsets kb + KW u
    bf16x8 wf[SKINNY_U][RT], af[SKINNY_U][MT];
  };
  auto load = [&](Batch& b, int kb) {
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) {
      const int k = kb + KW * u + 8 * lkg;
      const int kc = k < K - 8 ? k : K - 8;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) b.wf[u][rt] = *reinterpret_cast<const bf16x8*>(wrow[rt] + kc);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b.af[u][mt] = *reinterpret_cast<const bf16x8*>(arow[mt] + kc);
    }
  };
  auto multiply = [&](Batch& b, int kb) {
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) {
      // K and the range bounds are multiples of 8: a lane's 8 elements are all in or all out
      const bool kok = kb + KW * u + 8 * g4 < k_hi;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b.af[u][mt] = to_mfma_order(b.af[u][mt], fetch_from);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        // the permute runs in every lane (a lane that skipped it could not be read by the others)
        const bf16x8 moved = to_mfma_order(b.wf[u][rt], fetch_from);
        const bf16x8 w = kok ? moved : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, b.af[u][mt], acc[rt][mt], 0, 0, 0);
      }
    }
  };
  constexpr int STEP = KW * SKINNY_U;
  int kb = k_lo + 32 * (wave % 4);  // the same in every lane of a wavefront: the branches on it are uniform
  {
    // Two batches take turns, so that a wavefront always has loads in flight: with one, every batch
    // waits out the memory's latency before the next is even asked for.  No load below stands under a
    // condition of its own: the compiler counts the loads in flight behind the one it waits for, and
    // where a load may or may not have been issued it waits for all of them, the other batch's included.
    Batch b0, b1;
    int batches = kb < k_hi ? (k_hi - kb + STEP - 1) / STEP : 0;  // of this wavefront
    if (AHEAD && wave == 0) ask_row<RT, EPI>(ahead, M, rope);
    // The rows' shares of the sums of squares are asked for first, by the workgroup's first 256 threads
    // together and all at once, then the first batch (from clamped addresses also where the wavefront
    // has none); the scales are worked out when the shares are there, with the batch still on its way.
    row_scales_to_lds<MT>(s_scale, norm, M, K, tid, [&] { load(b0, kb); });
    if (AHEAD && wave == 0) ask_epilogue<RT, EPI, false>(ahead, blockIdx.x * RT, out, ldc, M, N, rope, norm);
    while (batches >= 3) {
      load(b1, kb + STEP);
      multiply(b0, kb);
      load(b0, kb + 2 * STEP);
      multiply(b1, kb + STEP);
      kb += 2 * STEP;
      batches -= 2;
    }
    if (batches == 2) {
      load(b1, kb + STEP);
      multiply(b0, kb);
      multiply(b1, kb + STEP);
    } else if (batches == 1) {
      multiply(b0, kb);
    }
  }

  // The four wavefronts' sums are added in wavefront order.  With one column tile wavefront 0 adds
  // and writes; with more, wavefront w takes column tile w, so that the epilogues run side by side.
  if (MT == 1) {
    if (wave > 0) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_part[wave - 1][rt * 4 + i][lane] = acc[rt][0][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][0][i] += s_part[w][rt * 4 + i][lane];
    if (NW == 16) {  // the other three ranges: each added up in wavefront order, then onto the first in range order
#pragma unroll
      for (int range = 1; range < 4; ++range)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float sum = s_part[4 * range - 1][rt * 4 + i][lane];
#pragma unroll
            for (int w = 0; w < 3; ++w) sum += s_part[4 * range + w][rt * 4 + i][lane];
            acc[rt][0][i] += sum;
          }
    }
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_part[wave][(rt * MT + mt) * 4 + i][lane] = acc[rt][mt][i];
    __syncthreads();
    if (wave >= MT) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      if (mt == wave) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float sum = s_part[0][(rt * MT + mt) * 4 + i][lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += s_part[w][(rt * MT + mt) * 4 + i][lane];
            acc[rt][mt][i] = sum;
          }
      }
  }

  float scale[MT];  // (the barrier above lies between the scales' writing and this)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) scale[mt] = s_scale[16 * mt + r];
  if (EPI != EPI_F32 && tickets.counters) {  // this wavefront's column tile: the sums of all k ranges, or done
    f32x4 mine[RT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      if (MT == 1 || mt == wave)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) mine[rt] = acc[rt][mt];
    if (!add_up_k_ranges<RT>(mine, blockIdx.x * MT + (MT > 1 ? wave : 0), blockIdx.y, gridDim.y, tickets)) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      if (MT == 1 || mt == wave)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][mt] = mine[rt];
  }
  skinny_epilogue<MT, RT, EPI>(acc, blockIdx.x * RT, MT > 1 ? wave : -1, out, ldc, bias, b_is_f32, M, N, blockIdx.y,
                               part_stride, rope, norm, scale, AHEAD ? &ahead : nullptr);
}

// The same product for 17..64 rows of A where there are many weight rows.  With several column
// tiles the kernel above is held up by the activations, which every workgroup reads again for its
// few weight rows, and by adding up its four wavefronts' sums.  Here a workgroup takes 64 RT weight
// rows, 16 RT per wavefront over the whole k range, and reads each slab of the activations (128 wide
// with RT = 2, 256 wide with RT = 1: the same weight bytes on their way) once: all threads load it together and leave it in LDS in the order the matrix instruction
// wants, where every wavefront reads its fragments with one 16-byte read each (two slabs take
// turns: the next is fetched while the current one is used).  Weight fragments come straight
// from memory as above.  Every wavefront ends with whole sums of its own rows.
template <int MT, int RT, int EPI, int WAVES = 4>
__global__ __launch_bounds__(64 * WAVES) void gemm_medium_kernel(void* __restrict__ out, int64_t ldc,
                                                          const bf16_t* __restrict__ A, int64_t lda,
                                                          const bf16_t* __restrict__ W,
                                                          const void* __restrict__ bias, int b_is_f32, int M,
                                                          int N, int K, int k_per_split, int64_t part_stride,
                                                          SkinnyRope rope, SkinnyTickets tickets, SkinnyNorm norm) {
  constexpr int KC = 256 / RT, CH = KC / 128;
  __shared__ bf16x8 a_lds[2][MT][KC / 32][PAE_WAVE];  // [slab][column tile][k step][lane]
  __shared__ float s_scale[16 * MT];                  // what the folded norm owes every row of A
  const int tid = threadIdx.x, lane = tid % PAE_WAVE, wave = tid / PAE_WAVE;
  const int g4 = lane / 16;
  const int tile_base = (blockIdx.x * WAVES + wave) * RT;  // this wavefront's first tile of 16 weight rows
  const bool stages = WAVES == 4 || tid < 256;           // the first four wavefronts bring the slabs of A
  const int k_lo = blockIdx.y * k_per_split;
  const int k_hi = min(K, k_lo + k_per_split);
  const int lrow = lane / 4, lkg = lane % 4;
  const int fetch_from = ((lane % 16) * 4 + lane / 16) * 4;
  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n = 16 * (tile_base + rt) + lrow;
    if (EPI == EPI_ROPE) {
      const int tile = tile_base + rt, per_head = rope.hd / 16;
      n = tile / per_head * rope.hd + rope_feature(tile % per_head, lrow, rope.rot);
    }
    wrow[rt] = W + (int64_t)(n < N ? n : N - 1) * K;  // rows past N are loaded from the last row and never stored
  }
  // the slab of A: thread t brings, per column tile, the 8 elements at k offset 8 (t % 16) of row
  // t / 16, which lane (t % 16) % 4 * 16 + t / 16 of k step (t % 16) / 4 wants as its B fragment
  const int arow = tid / 16, achunk = tid % 16;
  const bf16_t* aptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + arow;
    aptr[mt] = A + (int64_t)(m < M ? m : M - 1) * lda;
  }
  const int a_slot = (achunk % 4) * 16 + arow, a_step = achunk / 4;

  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {};
  struct Slab {
    bf16x8 wf[KC / 32][RT], a[MT][CH];
  };
  auto load = [&](Slab& b, int kc) {  // loads are unconditional, from clamped addresses
    if (stages)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int ka = kc + 128 * c + 8 * achunk;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) b.a[mt][c] = *reinterpret_cast<const bf16x8*>(aptr[mt] + (ka < K - 8 ? ka : K - 8));
      }
#pragma unroll
    for (int st = 0; st < KC / 32; ++st) {
      const int k = kc + 32 * st + 8 * lkg;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) b.wf[st][rt] = *reinterpret_cast<const bf16x8*>(wrow[rt] + (k < K - 8 ? k : K - 8));
    }
  };
  auto stage = [&](const Slab& b, int buf) {
    if (stages)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < CH; ++c) a_lds[buf][mt][4 * c + a_step][a_slot] = b.a[mt][c];
  };
  auto multiply = [&](Slab& b, int kc, int buf) {
#pragma unroll
    for (int st = 0; st < KC / 32; ++st) {
      // a lane past the end of the k range zeroes its weight fragment (K and the bounds are multiples of 8)
      const bool kok = kc + 32 * st + 8 * g4 < k_hi;
      bf16x8 af[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt] = a_lds[buf][mt][st][lane];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const bf16x8 moved = to_mfma_order(b.wf[st][rt], fetch_from);  // in every lane
        const bf16x8 w = kok ? moved : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, af[mt], acc[rt][mt], 0, 0, 0);
      }
    }
  };
  // The k range is the same for the whole workgroup: every wavefront passes the same barriers.  Two slabs
  // take turns; no load stands under a condition of its own (the compiler counts the loads in flight
  // behind the one it waits for, and where one may or may not have been issued it waits for all).
  Slab s0, s1;
  int kc = k_lo;
  int slabs = (k_hi - k_lo + KC - 1) / KC;  // at least one
  // the rows' shares of the sums of squares are asked for first, all at once, then the first slab
  row_scales_to_lds<MT>(s_scale, norm, M, K, tid, [&] { load(s0, kc); });
  stage(s0, 0);
  __syncthreads();
  while (slabs >= 3) {
    load(s1, kc + KC);
    multiply(s0, kc, 0);
    stage(s1, 1);
    __syncthreads();
    load(s0, kc + 2 * KC);
    multiply(s1, kc + KC, 1);
    stage(s0, 0);
    __syncthreads();
    kc += 2 * KC;
    slabs -= 2;
  }
  if (slabs == 2) {
    load(s1, kc + KC);
    multiply(s0, kc, 0);
    stage(s1, 1);
    __syncthreads();
    multiply(s1, kc + KC, 1);
  } else {
    multiply(s0, kc, 0);
  }
  float scale[MT];  // (written before the first barrier above)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) scale[mt] = s_scale[16 * mt + lane % 16];
  if (EPI != EPI_F32 && tickets.counters) {  // this wavefront's rows: the sums of all k ranges, or done
    if (!add_up_k_ranges<RT * MT>(reinterpret_cast<f32x4(&)[RT * MT]>(acc), blockIdx.x * WAVES + wave, blockIdx.y,
                                  gridDim.y, tickets))
      return;
  }
  skinny_epilogue<MT, RT, EPI>(acc, tile_base, -1, out, ldc, bias, b_is_f32, M, N, blockIdx.y, part_stride, rope, norm, scale);
}

// epilogue: 0 bfloat16 out (+bias), 1 float32 out (`splits` partials of `part_stride`
// elements each when splits > 1; a bias only with one split), 2 SiLU gate (N counts the
// interleaved gate and up rows, 8 and 8; out is [M, N / 2]), 3 rotation and cache write.
// Several k ranges of epilogues 0, 2 and 3 are added up inside the kernel (`tickets`).
// Which kernel runs is decided here from the sizes alone, by rules measured at the layer
// sizes of the 1.5B, 7B and 72B models.
static int launch_skinny(int epilogue, void* out, int64_t ldc, const void* A, int64_t lda, const void* W,
                         const void* bias, int b_is_f32, int M, int N, int K, int splits, int64_t part_stride,
                         const SkinnyRope& rope, SkinnyTickets tickets, const SkinnyNorm& norm, hipStream_t stream) {
  PAE_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: M=%d is outside 0..64", M);
  PAE_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && lda % 8 == 0, "gemm_skinny: N=%d K=%d lda=%lld (K and lda must be multiples of 8)",
              N, K, (long long)lda);
  const bool ticketed = splits > 1 && epilogue != EPI_F32;
  PAE_REQUIRE(splits >= 1 && (!ticketed || (tickets.parts && tickets.counters)),
              "gemm_skinny: %d k ranges with epilogue %d need scratch for partial sums and tickets", splits, epilogue);
  PAE_REQUIRE(!(bias && splits > 1 && !ticketed), "gemm_skinny: a bias cannot be combined with partial sums");
  if (!ticketed) tickets = SkinnyTickets{nullptr, nullptr};
  PAE_REQUIRE(!norm.row_stats || norm.row_stat_tiles > 0, "gemm_skinny: a row scale needs its shares of the sums of squares");
  PAE_REQUIRE(epilogue != EPI_RESIDUAL || (norm.next_rows && norm.next_w && norm.next_stats && norm.ld_next >= N && !bias),
              "gemm_skinny: the residual epilogue needs the next rows, the next norm's weight and room for its sums, and takes no bias");
  PAE_REQUIRE(epilogue != EPI_SWIGLU || (N % 16 == 0 && ldc % 4 == 0), "gemm_skinny: gated epilogue needs N %% 16 == 0, got %d", N);
  if (M == 0) return 0;
  // weight rows per workgroup: 16 for up to 8 rows of A, else 32, so that the activations, which every
  // workgroup re-reads, stay behind the weights (9 to 16 rows with 32: 7B gate/up at 16 rows 70.6 -> 63.5 us,
  // 32B 148.6 -> 135.8, 72B down 128.5 -> 108.6 us; at 8 rows and below 16 are as fast or faster at most
  // sizes), unless that leaves too few workgroups (the QKV product of the 1.5B sizes at 16 rows: 64
  // workgroups, 9.2 us).  5 to 8 rows with 32 only where there are very many weight rows (gate/up at 8
  // rows: 7B, 1,184 such workgroups, 61.1 -> 57.9 us, 32B, 1,728, 129.0 -> 123.2; but 1.5B, 560, 14.2 -> 15.0,
  // 14B, 864, 67.0 -> 67.6; at 4 rows and below never ahead; not with several k ranges: the 72B QKV product
  // in four ranges, 1,280 such workgroups, 40.4 -> 60.2 us).  Never with k ranges of 8,192 and more: 72B
  // gate/up, whose rows lie 16 KB apart, takes 195.9 us at 9 rows with 16 and 243.9 us with 32.
  const int mt = (M + 15) / 16;
  const int64_t groups32 = (int64_t)((N + 31) / 32) * splits;
  const bool long_ranges = (K + splits - 1) / splits >= 8192;
  const int rt = mt >= 2 || (!long_ranges && ((M > 8 && groups32 >= 128) || (M > 4 && splits == 1 && groups32 >= 1024))) ? 2 : 1;
  int k_per_split = (K + splits - 1) / splits;
  k_per_split = (k_per_split + 127) / 128 * 128;
  PAE_REQUIRE((int64_t)k_per_split * (splits - 1) < K, "gemm_skinny: %d k ranges are too many for K=%d", splits, K);
  // many weight rows and more than 16 rows of A: 128 weight rows a workgroup, activations through LDS
  // (measured at 1.5B/7B/72B layer sizes: ahead from about one workgroup per compute unit on, behind below)
  const int medium_groups = (N + 127) / 128;
  // Up to 48 rows of A and fewer than four such workgroups per compute unit: 64 weight rows a workgroup
  // instead (gate/up of the 7B sizes at 32 rows: 77 -> 61 us; at 64 rows the activations' re-reading costs
  // more than the idle units, and with few weight rows, as at the 1.5B sizes, the first kernel stays ahead).
  const int narrow_groups = (N + 63) / 64;
  // (also where only the smaller workgroups fill the chip: down of the 7B sizes in 8 k ranges, 52 -> 48 us at 64 rows)
  const bool only_narrow_fills = (int64_t)medium_groups * splits < 256 && (int64_t)narrow_groups * splits >= 384;
  const bool wide = !only_narrow_fills &&
                    (mt > 3 || (int64_t)medium_groups * splits >= 1024 || (int64_t)narrow_groups * splits < 512);
  // (up to 16 rows every product takes the first kernel, whose order of adding the decode program shares:
  // a row's sums are then the same bits alone, in a batch, in a program or launched by itself)
  // One k range and 16 W weight rows a workgroup (W = 5 to 8 wavefronts of 16 rows each) where that many
  // workgroups are nearly as many as the chip's 256 compute units: every unit then streams its share of
  // the weights once, with no partial sums to write and fetch back (1.5B gate/up, 224 workgroups of 80
  // rows: at 32 rows 19.1 -> 16.7 us, at 64 rows 23.4 -> 22.2 us against three ticketed ranges of 128-row
  // workgroups; with 205 workgroups, 16,384 weight rows, it is no faster than those).
  const int waves = ((N + 15) / 16 + 255) / 256;  // wavefronts a workgroup for at most 256 workgroups
  const int few_groups = ((N + 15) / 16 + waves - 1) / waves;
  if (M > 16 && splits == 1 && waves >= 5 && waves <= 8 && few_groups >= 216 &&
      (epilogue == EPI_BF16 || epilogue == EPI_SWIGLU)) {
#define LAUNCH_FEW(MT, EPI, W)                                                                                   \
  gemm_medium_kernel<MT, 1, EPI, W><<<dim3(few_groups, 1), 64 * W, 0, stream>>>(                                  \
      out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W_, bias, b_is_f32, M, N, K, k_per_split, part_stride, rope, tickets, norm)
#define FEW_BY_W(MT, EPI)                     \
  switch (waves) {                            \
    case 5: LAUNCH_FEW(MT, EPI, 5); break;    \
    case 6: LAUNCH_FEW(MT, EPI, 6); break;    \
    case 7: LAUNCH_FEW(MT, EPI, 7); break;    \
    default: LAUNCH_FEW(MT, EPI, 8); break;   \
  }
#define FEW_BY_MT(EPI)                       \
  switch (mt) {                              \
    case 2: FEW_BY_W(2, EPI); break;         \
    case 3: FEW_BY_W(3, EPI); break;         \
    default: FEW_BY_W(4, EPI); break;        \
  }
    const void* W_ = W;
    if (epilogue == EPI_BF16) {
      FEW_BY_MT(EPI_BF16);
    } else {
      FEW_BY_MT(EPI_SWIGLU);
    }
#undef FEW_BY_MT
#undef FEW_BY_W
#undef LAUNCH_FEW
    return pae_check_launch("gemm_medium (one workgroup a compute unit)");
  }
  if (M > 16 && ((int64_t)medium_groups * splits >= 256 || only_narrow_fills)) {
    dim3 mgrid(wide ? medium_groups : (N + 63) / 64, splits);
#define LAUNCH_MEDIUM(MT, EPI)                                                                                   \
  if (wide)                                                                                                      \
    gemm_medium_kernel<MT, 2, EPI><<<mgrid, 256, 0, stream>>>(out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W,  \
                                                              bias, b_is_f32, M, N, K, k_per_split, part_stride, rope, tickets, norm); \
  else                                                                                                           \
    gemm_medium_kernel<MT, 1, EPI><<<mgrid, 256, 0, stream>>>(out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W,  \
                                                              bias, b_is_f32, M, N, K, k_per_split, part_stride, rope, tickets, norm)
#define MEDIUM_BY_MT(EPI)                       \
  switch (mt) {                                 \
    case 1: LAUNCH_MEDIUM(1, EPI); break;       \
    case 2: LAUNCH_MEDIUM(2, EPI); break;       \
    case 3: LAUNCH_MEDIUM(3, EPI); break;       \
    default: LAUNCH_MEDIUM(4, EPI); break;      \
  }
    switch (epilogue) {
      case EPI_BF16: MEDIUM_BY_MT(EPI_BF16); break;
      case EPI_F32: MEDIUM_BY_MT(EPI_F32); break;
      case EPI_SWIGLU: MEDIUM_BY_MT(EPI_SWIGLU); break;
      case EPI_ROPE: MEDIUM_BY_MT(EPI_ROPE); break;
      case EPI_RESIDUAL: MEDIUM_BY_MT(EPI_RESIDUAL); break;
      default: return pae_fail("gemm_skinny: unknown epilogue %d", epilogue);
    }
#undef MEDIUM_BY_MT
#undef LAUNCH_MEDIUM
    return pae_check_launch("gemm_medium");
  }
  // Very few weight rows (the QKV product of the 1.5B sizes: 64 workgroups of 32 rows): the rows of A are
  // shared out too, 16 to a workgroup of the one-tile kernel, and the weights are read once from HBM and
  // again from L2 (1.5B QKV at 64 rows 10.5 -> 6.7 us; from about 100 workgroups on it is slower).
  if (mt >= 2 && !ticketed && (int64_t)((N + 31) / 32) * splits <= 96) {
    dim3 tiled((N + 15) / 16, splits, mt);
#define LAUNCH_TILED(EPI)                                                                                        \
  gemm_skinny_kernel<1, 1, EPI, 4><<<tiled, 256, 0, stream>>>(out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, bias, \
                                                               b_is_f32, M, N, K, k_per_split, part_stride, rope, tickets, norm)
    switch (epilogue) {
      case EPI_BF16: LAUNCH_TILED(EPI_BF16); break;
      case EPI_F32: LAUNCH_TILED(EPI_F32); break;
      case EPI_SWIGLU: LAUNCH_TILED(EPI_SWIGLU); break;
      case EPI_ROPE: LAUNCH_TILED(EPI_ROPE); break;
      case EPI_RESIDUAL: LAUNCH_TILED(EPI_RESIDUAL); break;
      default: return pae_fail("gemm_skinny: unknown epilogue %d", epilogue);
    }
#undef LAUNCH_TILED
    return pae_check_launch("gemm_skinny (rows of A in tiles)");
  }
  if (epilogue == EPI_RESIDUAL && mt == 1 && splits == 4 && K >= 1024 && ((N + 15) / 16 >= 192 || 32 * (int64_t)K <= 65536)) {
    // Four k ranges side by side in one workgroup of sixteen wavefronts: no tickets, no trip to memory
    // for partial sums; few workgroups, but each keeps its compute unit's memory pipeline full.  Ahead
    // wherever the 16-row workgroups fill the chip or have little to read each (1.5B O at 8 rows 7.2 ->
    // 5.9 us, 7B down 38.3 -> 36.1 us); the same bits as the ticketed ranges (see the kernel).
    gemm_skinny_kernel<1, 1, EPI_RESIDUAL, 4, 16><<<dim3((N + 15) / 16, 1), 1024, 0, stream>>>(
        out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, bias, b_is_f32, M, N, K, k_per_split, part_stride, rope,
        SkinnyTickets{nullptr, nullptr}, norm);
    return pae_check_launch("gemm_skinny (sixteen wavefronts)");
  }
  dim3 grid((N + 16 * rt - 1) / (16 * rt), splits);
  // four k steps of loads in flight per wavefront: deeper prefetch costs registers and measured slower
#define LAUNCH(MT, RT, EPI)                                                                                  \
  gemm_skinny_kernel<MT, RT, EPI, (MT == 1 ? 4 : 2)><<<grid, 256, 0, stream>>>(out, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, \
                                                               bias, b_is_f32, M, N, K, k_per_split, part_stride, rope, tickets, norm)
#define BY_MT(EPI)                                                   \
  switch (mt) {                                                      \
    case 1: if (rt == 2) { LAUNCH(1, 2, EPI); } else { LAUNCH(1, 1, EPI); } break; \
    case 2: LAUNCH(2, 2, EPI); break;                                \
    case 3: LAUNCH(3, 2, EPI); break;                                \
    default: LAUNCH(4, 2, EPI); break;                               \
  }
  switch (epilogue) {
    case EPI_BF16: BY_MT(EPI_BF16); break;
    case EPI_F32: BY_MT(EPI_F32); break;
    case EPI_SWIGLU: BY_MT(EPI_SWIGLU); break;
    case EPI_ROPE: BY_MT(EPI_ROPE); break;
    case EPI_RESIDUAL: BY_MT(EPI_RESIDUAL); break;
    default: return pae_fail("gemm_skinny: unknown epilogue %d", epilogue);
  }
#undef BY_MT
#undef LAUNCH
  return pae_check_launch("gemm_skinny");
}

// row_stats (or null): the rows of A are bfloat16(x * w_norm) of a row x that is still to be divided
// by its root mean square; row_stats[m][0 .. row_stat_tiles) add up to sum(x^2) and the sums of row m
// are multiplied by rsqrt(that / K + row_eps).  Epilogue 4 adds the sums into the float32 `out`
// (the residual) in place and leaves bfloat16(out * next_w) in next_rows and the shares of the new
// rows' sums of squares in next_stats[M][(N + 15) / 16].
// Several k ranges with an epilogue other than float32 partial sums are added up inside the kernel:
// ticket_parts is scratch of pae_skinny_ticket_floats(M, N, splits) floats and ticket_counters holds
// pae_skinny_ticket_slots(M, N) ints that are zero before the call and zero after it.  Launches that
// share the counters must not overlap.
extern "C" int pae_gemm_skinny(int epilogue, void* out, int64_t ldc, const void* A, int64_t lda, const void* W,
                               const void* bias, int b_is_f32, int M, int N, int K, int splits,
                               int64_t part_stride, float* ticket_parts, int* ticket_counters,
                               const float* row_stats, int row_stat_tiles, float row_eps, void* next_rows,
                               int64_t ld_next, const void* next_w, int next_w_is_f32, float* next_stats,
                               hipStream_t stream) {
  PAE_REQUIRE(epilogue != EPI_ROPE, "gemm_skinny: the rotating epilogue has an entry point of its own");
  const SkinnyNorm norm{row_stats, row_stat_tiles, row_eps, (bf16_t*)next_rows, ld_next, next_w, next_w_is_f32, next_stats};
  return launch_skinny(epilogue, out, ldc, A, lda, W, bias, b_is_f32, M, N, K, splits, part_stride, SkinnyRope{},
                       SkinnyTickets{ticket_parts, ticket_counters}, norm, stream);
}

// Counters and scratch floats that `splits` k ranges of an [M, K] x [N, K]^T product need for their
// tickets, whichever kernel takes the product (one counter per wavefront that ends with whole sums of
// its own; its accumulators for every range).
extern "C" int pae_skinny_ticket_slots(int M, int N) { return (N + 15) / 16 * ((M + 15) / 16); }
extern "C" int64_t pae_skinny_ticket_floats(int M, int N, int splits) {
  return (int64_t)((N + 127) / 128) * 8 * ((M + 15) / 16) * splits * 4 * PAE_WAVE;
}

// q_out[M, nh * hd] = rotated queries of A * W^T (+ bias), W = [(nh + 2 nkv) * hd, K] holding the
// query, key and value projections in that order; rotated keys and raw values of every row go to
// slot block_tables[tok_seq[m]][positions[m] / bs] * bs + positions[m] % bs of the cache.  With
// nkv == 0 only queries are projected and nothing is stored.  rot == 0 (cos_sin null) rotates nothing;
// else cos_sin[m][i] = (cos, sin) of row m's angle for pair i < rot / 2.
extern "C" int pae_gemm_skinny_rope(void* q_out, int64_t ldq, const void* A, int64_t lda, const void* W,
                                    const void* bias, int b_is_f32, int M, int K, int nh, int nkv, int hd, int rot,
                                    const float* cos_sin, const int* positions, const int* tok_seq,
                                    const int* block_tables, int max_blocks, int bs, void* k_cache, void* v_cache,
                                    int splits, float* ticket_parts, int* ticket_counters, const float* row_stats,
                                    int row_stat_tiles, float row_eps, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && hd % 16 == 0, "gemm_skinny_rope: bad head sizes nh=%d nkv=%d hd=%d", nh, nkv, hd);
  PAE_REQUIRE(rot >= 0 && rot <= hd && rot % 16 == 0 && (rot == 0 || cos_sin),
              "gemm_skinny_rope: rotary_dim %d must be a multiple of 16 up to head_dim %d", rot, hd);
  PAE_REQUIRE(ldq >= (int64_t)nh * hd && ldq % 4 == 0, "gemm_skinny_rope: row stride %lld of the queries", (long long)ldq);
  PAE_REQUIRE(positions, "gemm_skinny_rope: positions are missing");
  PAE_REQUIRE(nkv == 0 || (bs > 0 && max_blocks > 0 && k_cache && v_cache && block_tables && tok_seq),
              "gemm_skinny_rope: the cache write needs tables and pools");
  SkinnyRope rope{cos_sin, positions, tok_seq, block_tables, (bf16_t*)k_cache, (bf16_t*)v_cache,
                  nh, nkv, hd, rot, max_blocks, bs};
  const SkinnyNorm norm{row_stats, row_stat_tiles, row_eps, nullptr, 0, nullptr, 0, nullptr};
  return launch_skinny(EPI_ROPE, q_out, ldq, A, lda, W, bias, b_is_f32, M, (nh + 2 * nkv) * hd, K, splits, 0, rope,
                       SkinnyTickets{ticket_parts, ticket_counters}, norm, stream);
}
