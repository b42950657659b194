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
// Weights are given transposed (B^T (S,d_in), C^T (d_out,S)) so that every MFMA fragment is one 16-byte piece; both
// travel through LDS so that the four waves of a workgroup share one fetch.
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

// NT: state tiles of 16 the instantiation holds registers for (S <= 16 NT).  Two workgroups share a compute unit (a
// workgroup's life is a chain of short barrier-separated phases, so one alone leaves the unit idle most of the time):
// at most 256 registers, and U without padding, 128 x S floats = 80 KB at S = 160.  Instead of a pad, the 16-byte slot
// of element (row, mode) is XOR-ed with bits 1..3 of the row, which keeps the 16 rows of a tile access on 16 different
// slots; the scan, one thread per mode, follows the same map.
template <bool FINAL, int NT>
__global__ void __launch_bounds__(256, NT <= 10 ? 2 : 1)   // beyond S = 160 one workgroup fills the LDS anyway
lds_seq_kernel(const bf16_t* __restrict__ x, const float* __restrict__ A, const bf16_t* __restrict__ BmT,
               const bf16_t* __restrict__ CmT, bf16_t* __restrict__ y, const float* __restrict__ carry,
               float* __restrict__ Eout, int T, int Bt, int d_in, int S, int d_out) {
  extern __shared__ __align__(16) float Us[];       // LSQ_TB x S
  const int ldu = S;
  auto uslot = [](int row, int slot) { return slot ^ ((row >> 1) & 7); };   // 16-byte slot of a row (S/4 slots, a multiple of 8)
  const int blk = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, g = lane >> 4;
  const int t0 = blk * LSQ_TB;
  const int nvalid = min(LSQ_TB, T - t0);
  const int nt = S >> 4;
  // ---- U = X_blk B: wave w owns positions 32w .. 32w+31 (two tiles of 16).  The four waves need the same weight
  // fragments: B^T travels through LDS in chunks of 64 k (S rows of 128 bytes, 16-byte pieces XOR-ed with bits of the
  // row so that the 16 rows of a fragment read fall into 16 different slots), double-buffered in the space that U
  // takes afterwards, so a workgroup fetches every weight once instead of once per wave (a compute unit's
  // vector-memory path, not HBM or the matrix cores, is what this kernel runs against).
  {
    unsigned char* wst = (unsigned char*)Us;                 // two stages of S * 128 bytes
    const unsigned wstage = (unsigned)S * 128u;
    const int npiece = S * 8;                                // 16-byte pieces per chunk
    constexpr int WPT = (NT * 16 * 8 + 255) / 256;    // pieces per thread at the largest S
    floatx4_t acc[2][NT];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int n = 0; n < NT; ++n) acc[m][n] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    const bf16_t* xr[2];
    bool xok[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int t = t0 + 32 * w + 16 * m + r;
      xok[m] = t < T;
      xr[m] = x + ((size_t)(xok[m] ? t : 0) * Bt + b) * d_in + g * 8;
    }
    auto wload = [&](int k0, uint4 (&v)[WPT]) {
#pragma unroll
      for (int i = 0; i < WPT; ++i) {
        const int q = tid + i * 256, row = q >> 3, c = q & 7;
        v[i] = (q < npiece && k0 + c * 8 < d_in) ? *(const uint4*)(BmT + (size_t)row * d_in + k0 + c * 8) : make_uint4(0, 0, 0, 0);
      }
    };
    auto wstore = [&](int stage, const uint4 (&v)[WPT]) {
#pragma unroll
      for (int i = 0; i < WPT; ++i) {
        const int q = tid + i * 256, row = q >> 3, c = q & 7;
        if (q < npiece) *(uint4*)(wst + stage * wstage + row * 128 + ((c ^ ((row >> 1) & 7)) << 4)) = v[i];
      }
    };
    auto xload = [&](int k0, uint4 (&v)[2][2]) {             // the two k steps of a chunk, both position tiles
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int m = 0; m < 2; ++m)
          v[kk][m] = (xok[m] && k0 + 32 * kk < d_in) ? *(const uint4*)(xr[m] + k0 + 32 * kk) : make_uint4(0, 0, 0, 0);
    };
    // chunks are requested two iterations before the iteration that moves them to LDS (one iteration of MFMAs is
    // shorter than a trip to memory): wv0 / wv1 and xb / xc hold the next two chunks
    uint4 wv0[WPT], wv1[WPT], xa[2][2], xb[2][2], xc[2][2];
    wload(0, wv0);
    xload(0, xa);
    wload(64, wv1);
    xload(64, xb);
    wstore(0, wv0);
    wload(128, wv0);
    xload(128, xc);
    __syncthreads();
    // one pass: multiply chunk k0 from stage `cur`, move chunk k0+64 (registers NXT) to the other stage, request
    // chunk k0+192 into those registers
#define LSQ_PASS(NXT)                                                                                         \
    {                                                                                                         \
      const unsigned char* ws = wst + cur * wstage;                                                           \
      _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) {                                                      \
        _Pragma("unroll") for (int n = 0; n < NT; ++n) {                                                      \
          if (n < nt) {                                                                                       \
            const int row = 16 * n + r, c = kk * 4 + g;                                                       \
            const uint4 wa = *(const uint4*)(ws + row * 128 + ((c ^ ((row >> 1) & 7)) << 4));                 \
            acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa), as_bf16x8(xa[kk][0]), acc[0][n], 0, 0, 0); \
            acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa), as_bf16x8(xa[kk][1]), acc[1][n], 0, 0, 0); \
          }                                                                                                   \
        }                                                                                                     \
      }                                                                                                       \
      if (k0 + 64 < d_in) wstore(cur ^ 1, NXT);                                                               \
      wload(k0 + 192, NXT);                                                                                   \
      _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                                                        \
        _Pragma("unroll") for (int m = 0; m < 2; ++m) { xa[kk][m] = xb[kk][m]; xb[kk][m] = xc[kk][m]; }       \
      xload(k0 + 192, xc);                                                                                    \
      __syncthreads();                                                                                        \
      cur ^= 1;                                                                                               \
      k0 += 64;                                                                                               \
    }
    int cur = 0, k0 = 0;
    while (k0 < d_in) {
      LSQ_PASS(wv1)
      if (k0 < d_in) LSQ_PASS(wv0)
    }
#undef LSQ_PASS
    // (the last barrier of the loop: every wave is through with the weight stages, U may overwrite them)
    // D layout: lane (r, g) holds modes 16n + 4g + i of position r of the tile
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int n = 0; n < NT; ++n)
        if (n < nt)
          *(float4*)(Us + (size_t)(32 * w + 16 * m + r) * ldu + 4 * uslot(32 * w + 16 * m + r, 4 * n + g)) = make_float4(acc[m][n][0], acc[m][n][1], acc[m][n][2], acc[m][n][3]);
  }
  __syncthreads();
  // ---- scan over the block's positions: thread = mode
  if (tid < S) {
    const float a = A[tid];
    float h = FINAL ? carry[((size_t)blk * Bt + b) * S + tid] : 0.f;
    // element (p, tid) sits at p * ldu + 4 * uslot(p, tid / 4) + tid % 4
    auto at = [&](int p_) { return Us + (size_t)p_ * ldu + 4 * uslot(p_, tid >> 2) + (tid & 3); };
    int p = 0;
    for (; p + 8 <= nvalid; p += 8) {
      float u[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) u[i] = *at(p + i);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        h = fmaf(a, h, u[i]);
        if (FINAL) *at(p + i) = h;
      }
    }
    for (; p < nvalid; ++p) {
      h = fmaf(a, h, *at(p));
      if (FINAL) *at(p) = h;
    }
    if (!FINAL) Eout[((size_t)blk * Bt + b) * S + tid] = h;
  }
  if (!FINAL) return;
  __syncthreads();
  // ---- Y = H C: wave w, positions 32w .. 32w+31; H as bf16 head + remainder
  {
    constexpr int KS = (NT + 1) / 2;   // k steps of 32 modes this instantiation holds registers for
    const int ks2 = S >> 5;            // k steps of 32 modes (<= KS)
    uint4 hb[2][KS], lb[2][KS];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int hrow = 32 * w + 16 * m + r;
      const float* hr = Us + (size_t)hrow * ldu;
#pragma unroll
      for (int k = 0; k < KS; ++k) {
        if (k < ks2) {
          const float4 v0 = *(const float4*)(hr + 4 * uslot(hrow, 8 * k + 2 * g)), v1 = *(const float4*)(hr + 4 * uslot(hrow, 8 * k + 2 * g + 1));
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
    const int tA = t0 + 32 * w + r, tB = tA + 16;
    bf16_t* yA = y + ((size_t)min(tA, T - 1) * Bt + b) * d_out + 4 * g;
    bf16_t* yB = y + ((size_t)min(tB, T - 1) * Bt + b) * d_out + 4 * g;
    const int nto = d_out >> 4;
    // C^T travels through LDS like B^T above, 64 output features (4 tiles) at a time, double-buffered in the space of
    // U now that every wave holds its H fragments in registers.  Rows are S * 2 + 16 bytes: an odd number of 16-byte
    // slots, so the 16 rows of a fragment read fall into 16 different slots.
    __syncthreads();
    unsigned char* cst = (unsigned char*)Us;
    const unsigned RS = (unsigned)S * 2u + 16u, cstage = 64u * RS;
    const int ppr = S >> 3, npc = 64 * ppr;                  // 16-byte pieces per row and per stage
    constexpr int CPT = (64 * (NT * 16 / 8) + 255) / 256;
    auto cload = [&](int o0, uint4 (&v)[CPT]) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int q = tid + i * 256, row = q / ppr, c = q - row * ppr;
        v[i] = (q < npc && o0 + row < d_out) ? *(const uint4*)(CmT + (size_t)(o0 + row) * S + c * 8) : make_uint4(0, 0, 0, 0);
      }
    };
    auto cstore = [&](int stage, const uint4 (&v)[CPT]) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int q = tid + i * 256, row = q / ppr, c = q - row * ppr;
        if (q < npc) *(uint4*)(cst + stage * cstage + row * RS + c * 16) = v[i];
      }
    };
    uint4 cv0[CPT], cv1[CPT];     // the next two groups of output features
    cload(0, cv0);
    cload(64, cv1);
    cstore(0, cv0);
    cload(128, cv0);
    __syncthreads();
#define LSQ_OUT(NXT)                                                                                          \
    {                                                                                                         \
      const unsigned char* cs = cst + cur * cstage;                                                           \
      _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                         \
        const int ot = (o0 >> 4) + j;                                                                         \
        if (ot < nto) {                                                                                       \
          floatx4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};                                     \
          _Pragma("unroll") for (int k = 0; k < KS; ++k) {                                                    \
            if (k < ks2) {                                                                                    \
              const uint4 wc = *(const uint4*)(cs + (16 * j + r) * RS + (32 * k + 8 * g) * 2);                \
              a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc), as_bf16x8(hb[0][k]), a0, 0, 0, 0);  \
              a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc), as_bf16x8(lb[0][k]), a0, 0, 0, 0);  \
              a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc), as_bf16x8(hb[1][k]), a1, 0, 0, 0);  \
              a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wc), as_bf16x8(lb[1][k]), a1, 0, 0, 0);  \
            }                                                                                                 \
          }                                                                                                   \
          if (tA < T) *(uint2*)(yA + ot * 16) = make_uint2(pack2_bf16(a0[0], a0[1]), pack2_bf16(a0[2], a0[3])); \
          if (tB < T) *(uint2*)(yB + ot * 16) = make_uint2(pack2_bf16(a1[0], a1[1]), pack2_bf16(a1[2], a1[3])); \
        }                                                                                                     \
      }                                                                                                       \
      if (o0 + 64 < d_out) cstore(cur ^ 1, NXT);                                                              \
      cload(o0 + 192, NXT);                                                                                   \
      __syncthreads();                                                                                        \
      cur ^= 1;                                                                                               \
      o0 += 64;                                                                                               \
    }
    int cur = 0, o0 = 0;
    while (o0 < d_out) {
      LSQ_OUT(cv1)
      if (o0 < d_out) LSQ_OUT(cv0)
    }
#undef LSQ_OUT
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
  const size_t shm = (size_t)LSQ_TB * S * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(nblk, Bt);
#define LSQ_RUN(NTV)                                                                                                      \
  do {                                                                                                                    \
    static const hipError_t e1 = hipFuncSetAttribute((const void*)lds_seq_kernel<false, NTV>,                             \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);            \
    static const hipError_t e2 = hipFuncSetAttribute((const void*)lds_seq_kernel<true, NTV>,                              \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);            \
    if (e1 != hipSuccess || e2 != hipSuccess) {                                                                           \
      fstu_set_error("fstu_lds_sequence: hipFuncSetAttribute: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));       \
      return (int)(e1 != hipSuccess ? e1 : e2);                                                                           \
    }                                                                                                                     \
    hipLaunchKernelGGL((lds_seq_kernel<false, NTV>), grid, dim3(256), shm, s, (const bf16_t*)x, A, (const bf16_t*)BmT,    \
                       (const bf16_t*)CmT, (bf16_t*)y, (const float*)carry, E, T, Bt, d_in, S, d_out);                    \
    hipLaunchKernelGGL(lds_carry_kernel, dim3((unsigned)((BtS + 255) / 256)), dim3(256), 0, s, h, A, (const float*)E,     \
                       carry, nblk, T, (int)BtS, S);                                                                      \
    hipLaunchKernelGGL((lds_seq_kernel<true, NTV>), grid, dim3(256), shm, s, (const bf16_t*)x, A, (const bf16_t*)BmT,     \
                       (const bf16_t*)CmT, (bf16_t*)y, (const float*)carry, E, T, Bt, d_in, S, d_out);                    \
  } while (0)
  if (S <= 64) LSQ_RUN(4);
  else if (S <= 160) LSQ_RUN(10);
  else LSQ_RUN(16);
#undef LSQ_RUN
  FSTU_CHECK_LAUNCH("fstu_lds_sequence");
  return FSTU_OK;
}
