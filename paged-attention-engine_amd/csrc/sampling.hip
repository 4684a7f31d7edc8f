// Picking tokens from float32 logits: argmax (first maximum wins, as torch.argmax
// does in the reference, engine/scheduler.py:610) and inverse-CDF sampling from
// softmax(logits / temperature) with a uniform number per row that the host
// derives from (seed, request, token index).
//
// A row is cut into `chunks` contiguous chunks so that the vocabulary is read by
// many workgroups at once:
//   1. every chunk finds its maximum (and where it first occurs);
//   2. (only if a row samples) every chunk sums exp((x - row max) / T) in double,
//      thread by thread over contiguous segments and then segment by segment, so
//      that the sums follow index order;
//   3. one workgroup per row picks the first maximum, or finds the chunk, the
//      segment and the index at which the cumulative sum first exceeds u * total,
//      repeating step 2's additions exactly.
// Every sum runs in a fixed order, so a row's token does not depend on the batch.
#include "common.h"
#include "api.h"

#define SAMPLE_NT 256

__device__ __forceinline__ void chunk_bounds(int vocab, int chunks, int c, int& lo, int& hi, int& per) {
  const int size = (vocab + chunks - 1) / chunks;
  lo = min(c * size, vocab);
  hi = min(lo + size, vocab);
  per = (size + SAMPLE_NT - 1) / SAMPLE_NT;  // elements of a thread's contiguous segment
}

__global__ __launch_bounds__(SAMPLE_NT) void sample_chunk_max_kernel(float* __restrict__ chunk_max,
                                                                     int* __restrict__ chunk_arg,
                                                                     const float* __restrict__ logits, int64_t ld,
                                                                     int vocab, int chunks) {
  __shared__ float s_val[SAMPLE_NT];
  __shared__ int s_idx[SAMPLE_NT];
  const int c = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
  int lo, hi, per;
  chunk_bounds(vocab, chunks, c, lo, hi, per);
  const float* row = logits + (int64_t)r * ld;
  float best = -INFINITY;
  int best_i = -1;
  for (int i = lo + tid; i < hi; i += SAMPLE_NT) {  // ascending per thread: strict > keeps the first
    const float x = row[i];
    if (best_i < 0 || x > best) { best = x; best_i = i; }
  }
  s_val[tid] = best;
  s_idx[tid] = best_i;
  __syncthreads();
  for (int step = SAMPLE_NT / 2; step > 0; step >>= 1) {
    if (tid < step) {
      const float ov = s_val[tid + step];
      const int oi = s_idx[tid + step];
      const int mi = s_idx[tid];
      if (oi >= 0 && (mi < 0 || ov > s_val[tid] || (ov == s_val[tid] && oi < mi))) { s_val[tid] = ov; s_idx[tid] = oi; }
    }
    __syncthreads();
  }
  if (tid == 0) {
    chunk_max[r * chunks + c] = s_val[0];
    chunk_arg[r * chunks + c] = s_idx[0];
  }
}

// Sum of exp((x - row_max) * inv_t) over this thread's contiguous segment of the chunk.
__device__ __forceinline__ double segment_sum(const float* row, int lo, int hi, int per, int tid, float row_max,
                                              float inv_t) {
  const int a = min(lo + tid * per, hi), b = min(a + per, hi);
  double sum = 0.0;
  for (int i = a; i < b; ++i) sum += (double)expf((row[i] - row_max) * inv_t);
  return sum;
}

__device__ __forceinline__ float row_maximum(const float* chunk_max, int r, int chunks) {
  float m = chunk_max[r * chunks];
  for (int c = 1; c < chunks; ++c) m = fmaxf(m, chunk_max[r * chunks + c]);
  return m;
}

__global__ __launch_bounds__(SAMPLE_NT) void sample_chunk_sum_kernel(double* __restrict__ chunk_sum,
                                                                     const float* __restrict__ chunk_max,
                                                                     const float* __restrict__ logits, int64_t ld,
                                                                     const float* __restrict__ temperature,
                                                                     int vocab, int chunks) {
  __shared__ double s_seg[SAMPLE_NT];
  const int c = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
  const float temp = temperature[r];
  if (!(temp > 0.f)) return;
  int lo, hi, per;
  chunk_bounds(vocab, chunks, c, lo, hi, per);
  const float* row = logits + (int64_t)r * ld;
  s_seg[tid] = segment_sum(row, lo, hi, per, tid, row_maximum(chunk_max, r, chunks), 1.0f / temp);
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int t = 0; t < SAMPLE_NT; ++t) total += s_seg[t];
    chunk_sum[r * chunks + c] = total;
  }
}

__global__ __launch_bounds__(SAMPLE_NT) void sample_pick_kernel(int* __restrict__ tokens,
                                                                const float* __restrict__ chunk_max,
                                                                const int* __restrict__ chunk_arg,
                                                                const double* __restrict__ chunk_sum,
                                                                const float* __restrict__ logits, int64_t ld,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform, int vocab,
                                                                int chunks) {
  __shared__ double s_seg[SAMPLE_NT];
  __shared__ double s_before;
  __shared__ int s_where;
  __shared__ float s_cmax[128];
  __shared__ int s_carg[128];
  __shared__ double s_csum[128];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float temp = temperature ? temperature[r] : 0.f;
  // the chunks' results come in with one load per thread; one thread then walks them in index order
  if (tid < chunks) {
    s_cmax[tid] = chunk_max[r * chunks + tid];
    s_carg[tid] = chunk_arg[r * chunks + tid];
    if (temp > 0.f) s_csum[tid] = chunk_sum[r * chunks + tid];
  }
  __syncthreads();
  if (!(temp > 0.f)) {  // the same for the whole workgroup
    // pairwise: the larger value wins, and among equal values the smaller index (the first maximum)
    if (tid >= chunks && tid < 128) {
      s_cmax[tid] = -INFINITY;
      s_carg[tid] = -1;
    }
    __syncthreads();
    for (int step = 64; step > 0; step >>= 1) {
      if (tid < step) {
        const float ov = s_cmax[tid + step], mv = s_cmax[tid];
        const int oi = s_carg[tid + step], mi = s_carg[tid];
        if (oi >= 0 && (mi < 0 || ov > mv || (ov == mv && oi < mi))) {
          s_cmax[tid] = ov;
          s_carg[tid] = oi;
        }
      }
      __syncthreads();
    }
    if (tid == 0) tokens[r] = s_carg[0];
    return;
  }
  const float* row = logits + (int64_t)r * ld;
  float row_max = s_cmax[0];
  for (int c = 1; c < chunks; ++c) row_max = fmaxf(row_max, s_cmax[c]);
  if (tid == 0) {
    double total = 0.0;
    for (int c = 0; c < chunks; ++c) total += s_csum[c];
    const double target = (double)uniform[r] * total;
    double run = 0.0;
    int where = -1;
    for (int c = 0; c < chunks; ++c) {
      const double v = s_csum[c];
      if (run + v > target) { where = c; break; }
      run += v;
    }
    s_where = where;
    s_before = target - run;  // what is left to cover inside the chunk
    if (where < 0) tokens[r] = vocab - 1;  // u * total rounded up to the total
  }
  __syncthreads();
  const int c = s_where;
  if (c < 0) return;
  int lo, hi, per;
  chunk_bounds(vocab, chunks, c, lo, hi, per);
  const float inv_t = 1.0f / temp;
  s_seg[tid] = segment_sum(row, lo, hi, per, tid, row_max, inv_t);
  __syncthreads();
  if (tid == 0) {
    const double target = s_before;
    double run = 0.0;
    int seg = SAMPLE_NT - 1;
    for (int t = 0; t < SAMPLE_NT; ++t) {
      if (run + s_seg[t] > target) { seg = t; break; }
      run += s_seg[t];
    }
    const int a = min(lo + seg * per, hi), b = min(a + per, hi);
    int pick = b - 1 >= a ? b - 1 : hi - 1;
    for (int i = a; i < b; ++i) {
      run += (double)expf((row[i] - row_max) * inv_t);
      if (run > target) { pick = i; break; }
    }
    tokens[r] = pick;
  }
}

extern "C" int pae_sample_chunks(int vocab) {
  const int chunks = (vocab + 1023) / 1024;
  return chunks < 1 ? 1 : (chunks > 128 ? 128 : chunks);
}

// Workspace: chunk_max and chunk_arg hold num_rows * pae_sample_chunks(vocab) values,
// chunk_sum as many doubles (needed only with temperatures).
extern "C" int pae_sample(int* tokens, const float* logits, int64_t ld, const float* temperature,
                          const float* uniform, int num_rows, int vocab, float* chunk_max, int* chunk_arg,
                          double* chunk_sum, hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d V=%d ld=%lld", num_rows,
              vocab, (long long)ld);
  PAE_REQUIRE(!temperature || (uniform && chunk_sum), "sample: temperatures need uniform numbers and sums");
  PAE_REQUIRE(num_rows <= 65535, "sample: %d rows exceed the grid", num_rows);
  if (num_rows == 0) return 0;
  const int chunks = pae_sample_chunks(vocab);
  dim3 grid(chunks, num_rows);
  sample_chunk_max_kernel<<<grid, SAMPLE_NT, 0, stream>>>(chunk_max, chunk_arg, logits, ld, vocab, chunks);
  if (temperature)
    sample_chunk_sum_kernel<<<grid, SAMPLE_NT, 0, stream>>>(chunk_sum, chunk_max, logits, ld, temperature, vocab,
                                                            chunks);
  sample_pick_kernel<<<num_rows, SAMPLE_NT, 0, stream>>>(tokens, chunk_max, chunk_arg, chunk_sum, logits, ld,
                                                         temperature, uniform, vocab, chunks);
  return pae_check_launch("sample");
}

// ---------------------------------------------------------------------------------------------
// pae_sample_static: the same three kernels with their chunk results in a buffer that is part of
// the library's image on every GPU, so that the call allocates nothing (see api.h).
//
// Layout of the buffer: PAE_SAMPLE_STATIC_SLOTS doubles (chunk sums), then as many floats (chunk
// maxima), then as many ints (where each maximum first occurs).  A slot is one (row, chunk) pair.
// Nothing in it has to start at zero: every slot that a call reads, the same call has written
// before (maxima and places for every row, sums for the rows that sample), so what the call before
// left does not matter.  Calls that overlap on one GPU (two streams, two threads) share the buffer
// and race; callers run them one after the other.
#include <mutex>

#define PAE_SAMPLE_STATIC_BYTES (PAE_SAMPLE_STATIC_SLOTS * (sizeof(double) + sizeof(float) + sizeof(int)))
#define PAE_MAX_DEVICES 64

static __device__ __align__(256) unsigned char scratch[PAE_SAMPLE_STATIC_BYTES];

// The buffer's address on each device.  In host code `scratch` is only a handle for the runtime's
// symbol table: the address a kernel can use comes from hipGetSymbolAddress, once per device with
// that device current, because each GPU holds its own copy at its own address.
static void* g_scratch_of_device[PAE_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// The device a call works on is the one its stream belongs to (the null stream: the current device),
// not whichever device happens to be current: kernels launched on that stream run there, and each GPU
// has the buffer at an address of its own.
static int device_of_stream(hipStream_t stream, int* out) {
  int current = -1;
  hipError_t err = hipGetDevice(&current);
  if (err != hipSuccess) return pae_fail("sample_static: no current device: %s", hipGetErrorString(err));
  *out = current;
  if (stream) {
    hipDevice_t dev = -1;
    err = hipStreamGetDevice(stream, &dev);
    if (err != hipSuccess) return pae_fail("sample_static: cannot tell the stream's device: %s", hipGetErrorString(err));
    *out = (int)dev;
  }
  PAE_REQUIRE(*out >= 0 && *out < PAE_MAX_DEVICES, "sample_static: device %d beyond the %d this library keeps track of",
              *out, PAE_MAX_DEVICES);
  return 0;
}

// The buffer's address on device `dev`, looked up at the first call for that device with that device
// current (and the caller's device current again afterwards).  The lookup asks the runtime (it may load
// the code object there), so it must not fall inside a stream capture: `capturing` refuses it then.
static int scratch_on_device(int dev, bool capturing, void** out) {
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_of_device[dev]) {
    PAE_REQUIRE(!capturing, "sample_static: the first call on device %d falls inside a stream capture; call "
                "pae_sample_static_prepare (or pae_sample_static once) on this device before capturing", dev);
    int current = -1;
    hipError_t err = hipGetDevice(&current);
    if (err == hipSuccess && current != dev) err = hipSetDevice(dev);
    if (err != hipSuccess) return pae_fail("sample_static: cannot make device %d current: %s", dev, hipGetErrorString(err));
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (current != dev) (void)hipSetDevice(current);
    if (err != hipSuccess || !ptr)
      return pae_fail("sample_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(err));
    g_scratch_of_device[dev] = ptr;
  }
  *out = g_scratch_of_device[dev];
  return 0;
}

// Looks the buffer's address up for the current device, so that a later pae_sample_static there may
// be issued inside a stream capture.  Allocates nothing.
extern "C" int pae_sample_static_prepare() {
  int dev = -1;
  if (int code = device_of_stream(nullptr, &dev)) return code;
  void* base = nullptr;
  return scratch_on_device(dev, false, &base);
}

extern "C" int pae_sample_static_slots() { return PAE_SAMPLE_STATIC_SLOTS; }

extern "C" int pae_sample_static(int* tokens, const float* logits, int64_t ld, const float* temperature,
                                 const float* uniform, int num_rows, int vocab, hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && vocab > 0, "sample_static: bad sizes rows=%d V=%d", num_rows, vocab);
  const int64_t slots = (int64_t)num_rows * pae_sample_chunks(vocab);
  PAE_REQUIRE(slots <= PAE_SAMPLE_STATIC_SLOTS,
              "sample_static: %d rows of %d logits need %lld chunk slots, the built-in buffer holds %d "
              "(use pae_sample with a workspace of the caller's)",
              num_rows, vocab, (long long)slots, PAE_SAMPLE_STATIC_SLOTS);
  int dev = -1;
  if (int code = device_of_stream(stream, &dev)) return code;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (stream && hipStreamIsCapturing(stream, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
  void* base = nullptr;
  if (int code = scratch_on_device(dev, capture != hipStreamCaptureStatusNone, &base)) return code;
  double* chunk_sum = (double*)base;
  float* chunk_max = (float*)(chunk_sum + PAE_SAMPLE_STATIC_SLOTS);
  int* chunk_arg = (int*)(chunk_max + PAE_SAMPLE_STATIC_SLOTS);
  return pae_sample(tokens, logits, ld, temperature, uniform, num_rows, vocab, chunk_max, chunk_arg, chunk_sum,
                    stream);
}
