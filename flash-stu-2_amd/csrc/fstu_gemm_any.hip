// General dense contraction  C[m, n] = T( sum_k A[m, k] W[n, k] )  for what the bf16 prompt GEMM (fstu_gemm.hip) does
// not take: fp32 (the bit-parity path of the reference's fp32 configuration, flash_stu/model.py:108-205 with
// torch_dtype float32), bf16 shapes with K % 32 != 0 or unaligned rows, and operands with any pair of strides (the
// (K*d, T) slabs of the exact-mode operator in fp32, flash_stu/modules/stu.py:107-120; phi @ M_filters, stu.py:88).
// Accumulation in fp32 on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32; bf16 inputs widen exactly), one
// rounding to the output dtype.  A workgroup of 4 waves owns 64 rows x 64 features, a wave 32 x 32; K runs in tiles
// of 32 through LDS.  Every global access is bounds-checked, so any M, N, K >= 1 works.
#include "fstu_common.h"

namespace {

typedef float floatx16_t __attribute__((ext_vector_type(16)));
#define GA_BM 64
#define GA_BN 64
#define GA_BK 32
#define GA_LD (GA_BK + 1)

// rows x GA_BK tile of a strided matrix into LDS as fp32, zero beyond the edges; threads run along the index whose
// stride is 1 so that the loads coalesce either way
template <typename T>
__device__ __forceinline__ void ga_load_tile(float (*dst)[GA_LD], const T* __restrict__ src, long long srow, long long sk,
                                             int row0, int nrows, int k0, int K) {
#pragma unroll
  for (int i = 0; i < GA_BM * GA_BK / 256; ++i) {
    const int idx = threadIdx.x + 256 * i;
    int r, k;
    if (sk == 1) { k = idx % GA_BK; r = idx / GA_BK; }
    else { r = idx % GA_BM; k = idx / GA_BM; }
    const bool ok = row0 + r < nrows && k0 + k < K;
    dst[r][k] = ok ? DT<T>::ld(src + (size_t)(row0 + r) * srow + (size_t)(k0 + k) * sk) : 0.f;
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
gemm_any_kernel(const T* __restrict__ A, long long sam, long long sak, const T* __restrict__ W, long long swn, long long swk,
                T* __restrict__ C, long long ldc, int M, int N, int K) {
  __shared__ float xs[GA_BM][GA_LD], ws[GA_BN][GA_LD];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wm = w & 1, wn = w >> 1;
  const int m0 = blockIdx.x * GA_BM, n0 = blockIdx.y * GA_BN;
  const int l32 = lane & 31, lh = lane >> 5;
  floatx16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  for (int k0 = 0; k0 < K; k0 += GA_BK) {
    ga_load_tile<T>(xs, A, sam, sak, m0, M, k0, K);
    ga_load_tile<T>(ws, W, swn, swk, n0, N, k0, K);
    __syncthreads();
    // weights as the A operand (lane: feature l % 32, k = l / 32), activations as the B operand (lane: row l % 32)
#pragma unroll
    for (int kk = 0; kk < GA_BK; kk += 2)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ws[32 * wn + l32][kk + lh], xs[32 * wm + l32][kk + lh], acc, 0, 0, 0);
    __syncthreads();
  }
  // D: lane l holds row l % 32 and features 8*(e/4) + 4*(l/32) + e%4 of the wave's 32 x 32 tile
  const int m = m0 + 32 * wm + l32;
  if (m >= M) return;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int f = n0 + 32 * wn + 8 * (e >> 2) + 4 * lh + (e & 3);
    if (f < N) DT<T>::st(C + (size_t)m * ldc + f, acc[e]);
  }
}

}  // namespace

// C (M, N; row stride ldc) = T(A W^T) with A element (m, k) at A[m*sam + k*sak] and W element (n, k) at
// W[n*swn + k*swk] (strides in elements, any sign-free combination); fp32 accumulation, one rounding.
extern "C" int fstu_gemm_any(const void* A, int64_t sam, int64_t sak, const void* W, int64_t swn, int64_t swk, void* C,
                             int64_t ldc, int M, int N, int K, int dtype, void* stream) {
  FSTU_REQUIRE(A && W && C, FSTU_ENULL, "fstu_gemm_any: null pointer");
  FSTU_REQUIRE(M >= 1 && N >= 1 && K >= 1 && ldc >= N, FSTU_ESHAPE, "fstu_gemm_any: M=%d N=%d K=%d ldc=%lld", M, N, K, (long long)ldc);
  FSTU_REQUIRE(sam >= 0 && sak >= 0 && swn >= 0 && swk >= 0 && (sam > 0 || M == 1) && (sak > 0 || K == 1) && (swn > 0 || N == 1) &&
                   (swk > 0 || K == 1),
               FSTU_ESHAPE, "fstu_gemm_any: strides must be positive (sam=%lld sak=%lld swn=%lld swk=%lld)", (long long)sam,
               (long long)sak, (long long)swn, (long long)swk);
  const unsigned gx = (unsigned)((M + GA_BM - 1) / GA_BM), gy = (unsigned)((N + GA_BN - 1) / GA_BN);
  FSTU_REQUIRE(gy <= 65535u, FSTU_ESHAPE, "fstu_gemm_any: N=%d too large", N);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_gemm_any",
                      hipLaunchKernelGGL((gemm_any_kernel<T>), dim3(gx, gy), dim3(256), 0, (hipStream_t)stream, (const T*)A,
                                         (long long)sam, (long long)sak, (const T*)W, (long long)swn, (long long)swk, (T*)C,
                                         (long long)ldc, M, N, K));
  FSTU_CHECK_LAUNCH("fstu_gemm_any");
  return FSTU_OK;
}
