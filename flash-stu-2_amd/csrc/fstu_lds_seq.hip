// Dense LDS over a whole sequence on the matrix cores (bf16): the loop of mini_stu/lds.py:95-101,
//   h <- h * A + x_t @ B ;  y_t = T(h @ C),   t = 0 .. T-1, state h (Bt,S) fp32 carried,
// cut into blocks of 128 positions that run in parallel.  x_t @ B does not depend on the state, so a block forms
// U = X_blk B with MFMA tiles and scans it in LDS; the state that enters a block is handed over by a short chain:
//   pass 1  (block, batch row): U tile, scan from zero, the block's end state E
//   pass 2  per (row, mode): carry[k+1] = E[k] + A^len(k) * carry[k], carry[0] = the caller's h; the last carry is the
//           new h.  Splitting a sequence at a multiple of 128 therefore gives bit-identical states and outputs.
//   pass 3  (block, batch row): U tile again (x is read twice instead of writing and re-reading U: the same bytes,
//           no workspace of the size of the sequence), scan from carry[k], Y = H C with H split into a bf16 head and
//           a bf16 remainder so that the second product keeps the fp32 state's accuracy.
// Weights are given transposed (B^T (S,d_in), C^T (d_out,S)) so that every MFMA fragment is one 16-byte load.
#include <mutex>
#include "fstu_common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

#define LSQ_TB 128        // positions per block
#define LSQ_NTMAX 16      // state tiles of 16 (S <= 256)
#define LSQ_OOB 0xfffffff0u

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (unsigned)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 buf_load16(rsrc_t rs, unsigned off) {
  u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}

template <bool FINAL>
__global__ void __launch_bounds__(256)
lds_seq_kernel(const bf16_t* __restrict__ x, const float* __restrict__ A, const bf16_t* __restrict__ BmT,
               const bf16_t* __restrict__ CmT, bf16_t* __restrict__ y, const float* __restrict__ carry,
               float* __restrict__ Eout, int T, int Bt, int d_in, int S, int d_out) {
  extern __shared__ __align__(16) float Us[];       // LSQ_TB x (S + 4)
  const int ldu = S + 4;
  const int blk = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, g = lane >> 4;
  const int t0 = blk * LSQ_TB;
  const int nvalid = min(LSQ_TB, T - t0);
  const int nt = S >> 4;
  // ---- U = X_blk B: wave w owns positions 32w .. 32w+31 (two tiles of 16)
  {
    floatx4_t acc[2][LSQ_NTMAX];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int n = 0; n < LSQ_NTMAX; ++n) acc[m][n] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    // one descriptor per tile row: positions beyond T read zeros
    const bf16_t* xr[2];
    bool xok[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int t = t0 + 32 * w + 16 * m + r;
      xok[m] = t < T;
      xr[m] = x + ((size_t)(xok[m] ? t : 0) * Bt + b) * d_in + g * 8;
    }
    const bf16_t* br = BmT + (size_t)r * d_in + g * 8;
    // the x fragments of four k steps are in flight while the previous four are multiplied (rows of x lie Bt * d_in
    // elements apart: every fragment is a trip to memory of its own)
    constexpr int PF = 4;
    uint4 xn[PF][2];
#pragma unroll
    for (int u = 0; u < PF; ++u)
#pragma unroll
      for (int m = 0; m < 2; ++m) xn[u][m] = (xok[m] && 32 * u < d_in) ? *(const uint4*)(xr[m] + 32 * u) : make_uint4(0, 0, 0, 0);
    // weight fragments of the next k step are requested before the current one is multiplied
    uint4 wn[LSQ_NTMAX];
#pragma unroll
    for (int n = 0; n < LSQ_NTMAX; ++n) wn[n] = n < nt ? *(const uint4*)(br + (size_t)n * 16 * d_in) : make_uint4(0, 0, 0, 0);
    for (int k0 = 0; k0 < d_in; k0 += 32 * PF) {
      uint4 xb[PF][2];
#pragma unroll
      for (int u = 0; u < PF; ++u)
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          xb[u][m] = xn[u][m];
          const int kn = k0 + 32 * (PF + u);
          xn[u][m] = (xok[m] && kn < d_in) ? *(const uint4*)(xr[m] + kn) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        if (k0 + 32 * u < d_in) {
          uint4 wa[LSQ_NTMAX];
          const int kn = k0 + 32 * (u + 1);
#pragma unroll
          for (int n = 0; n < LSQ_NTMAX; ++n) {
            wa[n] = wn[n];
            if (n < nt) wn[n] = *(const uint4*)(br + (size_t)n * 16 * d_in + (kn < d_in ? kn : 0));
          }
#pragma unroll
          for (int n = 0; n < LSQ_NTMAX; ++n) {
            if (n < nt) {
              acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[n]), as_bf16x8(xb[u][0]), acc[0][n], 0, 0, 0);
              acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[n]), as_bf16x8(xb[u][1]), acc[1][n], 0, 0, 0);
            }
          }
        }
      }
    }
    // D layout: lane (r, g) holds modes 16n + 4g + i of position r of the tile
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int n = 0; n < LSQ_NTMAX; ++n)
        if (n < nt)
          *(float4*)(Us + (size_t)(32 * w + 16 * m + r) * ldu + 16 * n + 4 * g) = make_float4(acc[m][n][0], acc[m][n][1], acc[m][n][2], acc[m][n][3]);
  }
  __syncthreads();
  // ---- scan over the block's positions: thread = mode
  if (tid < S) {
    const float a = A[tid];
    float h = FINAL ? carry[((size_t)blk * Bt + b) * S + tid] : 0.f;
    float* col = Us + tid;
    int p = 0;
    for (; p + 8 <= nvalid; p += 8) {
      float u[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) u[i] = col[(size_t)(p + i) * ldu];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        h = fmaf(a, h, u[i]);
        if (FINAL) col[(size_t)(p + i) * ldu] = h;
      }
    }
    for (; p < nvalid; ++p) {
      h = fmaf(a, h, col[(size_t)p * ldu]);
      if (FINAL) col[(size_t)p * ldu] = h;
    }
    if (!FINAL) Eout[((size_t)blk * Bt + b) * S + tid] = h;
  }
  if (!FINAL) return;
  __syncthreads();
  // ---- Y = H C: wave w, positions 32w .. 32w+31; H as bf16 head + remainder
  {
    const int ks2 = S >> 5;        // k steps of 32 modes (<= 8)
    uint4 hb[2][8], lb[2][8];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const float* hr = Us + (size_t)(32 * w + 16 * m + r) * ldu + g * 8;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (k < ks2) {
          const float4 v0 = *(const float4*)(hr + 32 * k), v1 = *(const float4*)(hr + 32 * k + 4);
          const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
          unsigned hi[4], lo[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            hi[i] = pack2_bf16(v[2 * i], v[2 * i + 1]);
            lo[i] = pack2_bf16(v[2 * i] - __uint_as_float(hi[i] << 16), v[2 * i + 1] - __uint_as_float(hi[i] & 0xffff0000u));
          }
          hb[m][k] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
          lb[m][k] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        }
      }
    }
    const bf16_t* cr = CmT + (size_t)r * S + g * 8;
    const int tA = t0 + 32 * w + r, tB = tA + 16;
    bf16_t* yA = y + ((size_t)min(tA, T - 1) * Bt + b) * d_out + 4 * g;
    bf16_t* yB = y + ((size_t)min(tB, T - 1) * Bt + b) * d_out + 4 * g;
    const int nto = d_out >> 4;
    uint4 cn[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) cn[k] = k < ks2 ? *(const uint4*)(cr + 32 * k) : make_uint4(0, 0, 0, 0);
    for (int ot = 0; ot < nto; ++ot) {
      floatx4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
      uint4 wc[8];
      const int on = ot + 1 < nto ? ot + 1 : ot;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        wc[k] = cn[k];
        if (k < ks2) cn[k] = *(const uint4*)(cr + (size_t)on * 16 * S + 32 * k);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (k < ks2) {
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc[k]), as_bf16x8(hb[0][k]), a0, 0, 0, 0);
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc[k]), as_bf16x8(lb[0][k]), a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc[k]), as_bf16x8(hb[1][k]), a1, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc[k]), as_bf16x8(lb[1][k]), a1, 0, 0, 0);
        }
      }
      if (tA < T) *(uint2*)(yA + ot * 16) = make_uint2(pack2_bf16(a0[0], a0[1]), pack2_bf16(a0[2], a0[3]));
      if (tB < T) *(uint2*)(yB + ot * 16) = make_uint2(pack2_bf16(a1[0], a1[1]), pack2_bf16(a1[2], a1[3]));
    }
  }
}

// carry[0] = h; carry[k+1] = E[k] + A^len(k) * carry[k]; h = carry[nblk]
__global__ void __launch_bounds__(256)
lds_carry_kernel(float* __restrict__ h, const float* __restrict__ A, const float* __restrict__ E, float* __restrict__ carry,
                 int nblk, int T, int BtS, int S) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= BtS) return;
  const double a = (double)A[i % S];
  const float ap_full = (float)pow(a, (double)LSQ_TB);
  float c = h[i];
  carry[i] = c;
  for (int k = 0; k < nblk; ++k) {
    const int len = min(LSQ_TB, T - k * LSQ_TB);
    const float ap = len == LSQ_TB ? ap_full : (float)pow(a, (double)len);
    c = fmaf(ap, c, E[(size_t)k * BtS + i]);
    carry[(size_t)(k + 1) * BtS + i] = c;
  }
  h[i] = c;
}

}  // namespace

extern "C" size_t fstu_lds_sequence_ws_floats(int T, int Bt, int S) {
  if (T < 0 || Bt < 1 || S < 1) return 0;
  const size_t nblk = (size_t)(T + LSQ_TB - 1) / LSQ_TB;
  return (2 * nblk + 1) * (size_t)Bt * S;
}

extern "C" int fstu_lds_sequence(float* h, const void* x, const float* A, const void* BmT, const void* CmT, void* y, float* ws,
                                 int T, int Bt, int d_in, int S, int d_out, void* stream) {
  FSTU_REQUIRE(h && x && A && BmT && CmT && y && ws, FSTU_ENULL, "fstu_lds_sequence: null pointer");
  FSTU_REQUIRE(T >= 0 && Bt >= 1 && Bt <= 65535, FSTU_ESHAPE, "fstu_lds_sequence: T=%d Bt=%d", T, Bt);
  FSTU_REQUIRE(d_in >= 32 && d_in % 32 == 0 && S >= 32 && S % 32 == 0 && S <= 16 * LSQ_NTMAX && d_out >= 16 && d_out % 16 == 0,
               FSTU_ESHAPE, "fstu_lds_sequence: need d_in %% 32 == 0, S %% 32 == 0 (<= %d), d_out %% 16 == 0 (d_in=%d S=%d d_out=%d)",
               16 * LSQ_NTMAX, d_in, S, d_out);
  FSTU_REQUIRE(fstu_aligned(x, 16) && fstu_aligned(BmT, 16) && fstu_aligned(CmT, 16) && fstu_aligned(y, 8) && fstu_aligned(ws, 16),
               FSTU_EALIGN, "fstu_lds_sequence: pointers must be 16-byte aligned");
  if (T == 0) return FSTU_OK;
  const int nblk = (T + LSQ_TB - 1) / LSQ_TB;
  const size_t BtS = (size_t)Bt * S;
  float* carry = ws;
  float* E = ws + (size_t)(nblk + 1) * BtS;
  const size_t shm = (size_t)LSQ_TB * (S + 4) * sizeof(float);
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&]() {
    attr_err = hipFuncSetAttribute((const void*)lds_seq_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute((const void*)lds_seq_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
  });
  if (attr_err != hipSuccess) { fstu_set_error("fstu_lds_sequence: hipFuncSetAttribute: %s", hipGetErrorString(attr_err)); return (int)attr_err; }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(nblk, Bt);
  hipLaunchKernelGGL(lds_seq_kernel<false>, grid, dim3(256), shm, s, (const bf16_t*)x, A, (const bf16_t*)BmT, (const bf16_t*)CmT,
                     (bf16_t*)y, (const float*)carry, E, T, Bt, d_in, S, d_out);
  hipLaunchKernelGGL(lds_carry_kernel, dim3((unsigned)((BtS + 255) / 256)), dim3(256), 0, s, h, A, (const float*)E, carry, nblk, T,
                     (int)BtS, S);
  hipLaunchKernelGGL(lds_seq_kernel<true>, grid, dim3(256), shm, s, (const bf16_t*)x, A, (const bf16_t*)BmT, (const bf16_t*)CmT,
                     (bf16_t*)y, (const float*)carry, E, T, Bt, d_in, S, d_out);
  FSTU_CHECK_LAUNCH("fstu_lds_sequence");
  return FSTU_OK;
}
