// Picking tokens from float32 logits: argmax (first maximum wins, as torch.argmax
// does in the reference, engine/scheduler.py:610) and inverse-CDF sampling from
// softmax(logits / temperature) with a uniform number per row that the host
// derives from (seed, request, token index).  One block per row; every sum runs
// in a fixed order over the vocabulary, so a row's token does not depend on the
// other rows of the batch.
#include "common.h"
#include "api.h"

#define SAMPLE_NT 256

// tokens[r] = temperature[r] == 0 ? argmax : first index whose cumulative
// probability exceeds u[r] * total.
__global__ __launch_bounds__(SAMPLE_NT) void sample_kernel(int* __restrict__ tokens,
                                                           const float* __restrict__ logits, int64_t ld,
                                                           const float* __restrict__ temperature,
                                                           const float* __restrict__ uniform, int vocab) {
  __shared__ float s_max[SAMPLE_NT];
  __shared__ int s_idx[SAMPLE_NT];
  __shared__ double s_sum[SAMPLE_NT];
  __shared__ double s_target;
  __shared__ int s_segment;
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const float* row = logits + (int64_t)r * ld;
  // a contiguous segment of the vocabulary per thread, so prefix sums follow index order
  const int per = (vocab + SAMPLE_NT - 1) / SAMPLE_NT;
  const int lo = tid * per < vocab ? tid * per : vocab;
  const int hi = lo + per < vocab ? lo + per : vocab;

  float best = -INFINITY;
  int best_i = -1;
  for (int i = lo; i < hi; ++i) {
    const float x = row[i];
    if (best_i < 0 || x > best) { best = x; best_i = i; }
  }
  s_max[tid] = best;
  s_idx[tid] = best_i;
  __syncthreads();
  if (tid == 0) {  // segments in index order, strict comparison: the first maximum wins
    float b = s_max[0];
    int bi = s_idx[0];
    for (int w = 1; w < SAMPLE_NT; ++w)
      if (s_idx[w] >= 0 && s_max[w] > b) { b = s_max[w]; bi = s_idx[w]; }
    s_max[0] = b;
    s_idx[0] = bi;
  }
  __syncthreads();
  const float row_max = s_max[0];
  const int arg = s_idx[0];
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) tokens[r] = arg;
    return;
  }
  const float inv_t = 1.0f / temp;
  double part = 0.0;
  for (int i = lo; i < hi; ++i) part += (double)expf((row[i] - row_max) * inv_t);
  s_sum[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int w = 0; w < SAMPLE_NT; ++w) total += s_sum[w];
    const double target = (double)uniform[r] * total;
    double run = 0.0;
    int seg = -1;
    for (int w = 0; w < SAMPLE_NT; ++w) {
      const double v = s_sum[w];
      s_sum[w] = run;  // exclusive prefix
      if (seg < 0 && run + v > target) seg = w;
      run += v;
    }
    s_target = target;
    s_segment = seg;
    if (seg < 0) tokens[r] = vocab - 1;  // u * total rounded up to the total
  }
  __syncthreads();
  if (tid == s_segment) {
    double run = s_sum[tid];
    int pick = hi - 1;
    for (int i = lo; i < hi; ++i) {
      run += (double)expf((row[i] - row_max) * inv_t);
      if (run > s_target) { pick = i; break; }
    }
    tokens[r] = pick;
  }
}

extern "C" int pae_sample(int* tokens, const float* logits, int64_t ld, const float* temperature,
                          const float* uniform, int num_rows, int vocab, hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d V=%d ld=%lld", num_rows,
              vocab, (long long)ld);
  PAE_REQUIRE(!temperature || uniform, "sample: temperatures need uniform numbers");
  if (num_rows == 0) return 0;
  sample_kernel<<<num_rows, SAMPLE_NT, 0, stream>>>(tokens, logits, ld, temperature, uniform, vocab);
  return pae_check_launch("sample");
}
