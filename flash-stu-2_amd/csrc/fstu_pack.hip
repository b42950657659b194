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
