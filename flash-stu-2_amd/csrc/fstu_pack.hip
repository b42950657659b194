// Packing of bf16 weights into MFMA-fragment order for the decode kernels.
//
// Packed layout (built once on the host side from the (N,K) row-major weight):
//   Wp[tile][kstep][lane][8]   tile = n/16, kstep = k/32, lane = 16*g + r,
//   element e of lane (r,g) is W[16*tile + r][32*kstep + 8*g + e]
// i.e. exactly the A-operand fragment of v_mfma_f32_16x16x32_bf16, so one wave
// load instruction (64 lanes x 16 B) reads 1 KB of contiguous memory and a wave
// that walks a K range streams one contiguous block.  Rows beyond N are zero.
#include "fstu_common.h"

template <int DUMMY>
__global__ void pack_rows_kernel(const bf16_t* __restrict__ W, bf16_t* __restrict__ Wp, int N, int K, int ntiles) {
  // one thread per packed 16-byte fragment
  const size_t nfrag = (size_t)ntiles * (K >> 5) * 64;
  for (size_t f = (size_t)blockIdx.x * blockDim.x + threadIdx.x; f < nfrag; f += (size_t)gridDim.x * blockDim.x) {
    const int lane = f & 63;
    const size_t ts = f >> 6;
    const int kstep = ts % (K >> 5);
    const int tile = ts / (K >> 5);
    const int r = lane & 15, g = lane >> 4;
    const int n = tile * 16 + r;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n < N) v = *(const uint4*)(W + (size_t)n * K + kstep * 32 + g * 8);
    *(uint4*)(Wp + f * 8) = v;
  }
}

extern "C" int64_t fstu_packed_elems(int N, int K) { return (int64_t)((N + 15) / 16) * 16 * (int64_t)K; }

extern "C" int fstu_pack_rows(const void* W, void* Wp, int N, int K, void* stream) {
  FSTU_REQUIRE(W && Wp, FSTU_ENULL, "fstu_pack_rows: null pointer");
  FSTU_REQUIRE(N >= 1 && K >= 32 && K % 32 == 0, FSTU_ESHAPE, "fstu_pack_rows: N=%d K=%d (K must be a multiple of 32)", N, K);
  FSTU_REQUIRE(fstu_aligned(W, 16) && fstu_aligned(Wp, 16), FSTU_EALIGN, "fstu_pack_rows: pointers must be 16-byte aligned");
  const int ntiles = (N + 15) / 16;
  size_t nfrag = (size_t)ntiles * (K >> 5) * 64;
  unsigned blocks = (unsigned)((nfrag + 255) / 256 > 65535 ? 65535 : (nfrag + 255) / 256);
  hipLaunchKernelGGL(pack_rows_kernel<0>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)W, (bf16_t*)Wp, N,
                     K, ntiles);
  FSTU_CHECK_LAUNCH("fstu_pack_rows");
  return FSTU_OK;
}

// ---------------------------------------------------------------- transpose of the last two dimensions
// out[b][c][r] = in[b][r][c] through 64 x 64 tiles in LDS (rows padded by one 32-bit word so that the transposed reads
// fall into different banks): both the loads and the stores walk the contiguous dimension.  Used to hand a few long
// sequences to the spectral convolution time-major (flash_stu/modules/stu.py:89-98 of the reference convolves
// (B, L, d) tensors along L).
template <typename T>
__global__ void __launch_bounds__(256)
transpose_tiles_kernel(const T* __restrict__ in, T* __restrict__ out, int R, int C) {
  __shared__ T tile[64][64 + 4 / sizeof(T) * 1];
  const int b = blockIdx.z, r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int j = threadIdx.x & 63, i0 = threadIdx.x >> 6;
  const T* src = in + (size_t)b * R * C;
  T* dst = out + (size_t)b * R * C;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int i = i0 + 4 * k;
    if (r0 + i < R && c0 + j < C) tile[i][j] = src[(size_t)(r0 + i) * C + c0 + j];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int i = i0 + 4 * k;
    if (c0 + i < C && r0 + j < R) dst[(size_t)(c0 + i) * R + r0 + j] = tile[j][i];
  }
}

extern "C" int fstu_transpose(const void* in, void* out, int B, int R, int C, int dtype, void* stream) {
  FSTU_REQUIRE(in && out && in != out, FSTU_ENULL, "fstu_transpose: null or aliased pointers");
  FSTU_REQUIRE(B >= 1 && B <= 65535 && R >= 1 && C >= 1 && (R + 63) / 64 <= 65535, FSTU_ESHAPE, "fstu_transpose: B=%d R=%d C=%d", B, R, C);
  const dim3 grid((C + 63) / 64, (R + 63) / 64, B);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_transpose",
                      hipLaunchKernelGGL(transpose_tiles_kernel<T>, grid, dim3(256), 0, (hipStream_t)stream, (const T*)in, (T*)out, R, C));
  FSTU_CHECK_LAUNCH("fstu_transpose");
  return FSTU_OK;
}
