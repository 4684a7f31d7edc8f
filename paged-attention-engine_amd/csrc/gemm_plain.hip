// C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]): the plain matrix product of the
// float32 path, also available for bfloat16 operands with float32 accumulation.
//
// W is stored (out_features, in_features) row-major as in the checkpoint, the
// layout F.linear takes in the reference (engine/model.py:303-305,315,318-320).
// Products are accumulated with fused multiply-adds in float32, k ascending, in
// blocks of 512 of k whose sums are then added up in order (with rows of 30,000
// terms one running sum loses a digit more than the block sums do): no
// reduced-precision matrix mode, no split over k across threads, and the value
// of an output element does not depend on M, on the tile it falls in or on which
// other rows share the launch.
#include "common.h"
#include "api.h"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16
#define GP_BLOCK_TILES 32  // k tiles whose sum is formed before it joins the total: 512 of k

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_plain_kernel(TC* __restrict__ C, int64_t ldc,
                                                         const TA* __restrict__ A, int64_t lda,
                                                         const TA* __restrict__ W, const void* __restrict__ bias,
                                                         int b_is_f32, int M, int N, int K) {
  __shared__ float As[GP_BK][GP_BM + 4];
  __shared__ float Ws[GP_BK][GP_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GP_BM, n0 = blockIdx.x * GP_BN;
  const int lr = tid / 4;        // tile row this thread loads
  const int lk = (tid % 4) * 4;  // first of its four k
  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

  int tiles_in_block = 0;
  for (int k0 = 0; k0 < K; k0 += GP_BK) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + lk + u;
      const int am = m0 + lr, wn = n0 + lr;
      As[lk + u][lr] = (am < M && k < K) ? to_f32(A[(int64_t)am * lda + k]) : 0.f;
      Ws[lk + u][lr] = (wn < N && k < K) ? to_f32(W[(int64_t)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
    if (++tiles_in_block == GP_BLOCK_TILES) {
      tiles_in_block = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = total[i][j] + acc[i][j];
      if (bias) v += load_param(bias, b_is_f32, n);
      C[(int64_t)m * ldc + n] = from_f32<TC>(v);
    }
  }
}

// in_dtype: operands; out_dtype: C.  Supported: f32->f32, bf16->bf16, bf16->f32.
extern "C" int pae_gemm_plain(int in_dtype, int out_dtype, void* C, int64_t ldc, const void* A, int64_t lda,
                              const void* W, const void* bias, int b_is_f32, int M, int N, int K,
                              hipStream_t stream) {
  PAE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  PAE_REQUIRE(lda >= K && ldc >= N, "gemm: leading dimensions lda=%lld ldc=%lld too small for K=%d N=%d",
              (long long)lda, (long long)ldc, K, N);
  if (M == 0) return 0;
  dim3 grid((N + GP_BN - 1) / GP_BN, (M + GP_BM - 1) / GP_BM);
  PAE_REQUIRE(grid.y <= 65535, "gemm: M=%d exceeds the grid", M);
  if (in_dtype == PAE_F32 && out_dtype == PAE_F32)
    gemm_plain_kernel<float, float><<<grid, 256, 0, stream>>>((float*)C, ldc, (const float*)A, lda,
                                                              (const float*)W, bias, b_is_f32, M, N, K);
  else if (in_dtype == PAE_BF16 && out_dtype == PAE_BF16)
    gemm_plain_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)C, ldc, (const bf16_t*)A, lda,
                                                                (const bf16_t*)W, bias, b_is_f32, M, N, K);
  else if (in_dtype == PAE_BF16 && out_dtype == PAE_F32)
    gemm_plain_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((float*)C, ldc, (const bf16_t*)A, lda,
                                                               (const bf16_t*)W, bias, b_is_f32, M, N, K);
  else
    return pae_fail("gemm: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
  return pae_check_launch("gemm_plain");
}
