// Dense LDS over a whole sequence on the matrix cores (bf16): the loop of mini_stu/lds.py:95-101,
//   h <- h * A + x_t @ B ;  y_t = T(h @ C),   t = 0 .. T-1, state h (Bt,S) fp32 carried,
// cut into blocks of 128 positions that run in parallel, x read ONCE.  x_t @ B does not depend on the state, so a
// workgroup (block, batch row) forms U = X_blk B with MFMA tiles and keeps it in LDS from then on:
//   1  scan U from zero: the block's end state E, published at once as tagged 64-bit words (value, tag of the call)
//   2  the state that enters the block: carry = h, then carry = E[j] + A^128 * carry over the blocks j in front of it,
//      read from what those blocks published (they are earlier in launch order, so they are resident or done, and
//      they publish before they wait for anything: the wait ends; it is bounded all the same and reports a
//      time-out through a status word instead of hanging).  The chain is the same fused multiply-adds in the same
//      order for every block, so splitting a sequence at a multiple of 128 gives bit-identical states and outputs.
//      The last block of a row also forms the state behind the sequence.
//   3  scan U again from the carry (now the true states H), Y = H C with H split into a bf16 head and a bf16
//      remainder so that the second product keeps the fp32 state's accuracy.
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
#define LSQ_SPIN_LIMIT (1 << 18)   // polls of one batch of published states before the wait gives up
#define LSQ_LOOK 8                 // published states requested at a time

template <int NT>
__global__ void __launch_bounds__(256, NT <= 10 ? 2 : 1)   // beyond S = 160 one workgroup fills the LDS anyway
lds_seq_kernel(const bf16_t* __restrict__ x, const float* __restrict__ A, const bf16_t* __restrict__ BmT,
               const bf16_t* __restrict__ CmT, bf16_t* __restrict__ y, const float* __restrict__ h0,
               float* __restrict__ hnew, unsigned long long* __restrict__ etag, unsigned* __restrict__ status, unsigned tag,
               int T, int Bt, int d_in, int S, int d_out) {
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
    // element (p, tid) sits at p * ldu + 4 * uslot(p, tid / 4) + tid % 4
    auto at = [&](int p_) { return Us + (size_t)p_ * ldu + 4 * uslot(p_, tid >> 2) + (tid & 3); };
    // 1: the block's end state from zero, published as (tag, value)
    float e = 0.f;
    {
      int p = 0;
      for (; p + 8 <= nvalid; p += 8) {
        float u[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = *at(p + i);
#pragma unroll
        for (int i = 0; i < 8; ++i) e = fmaf(a, e, u[i]);
      }
      for (; p < nvalid; ++p) e = fmaf(a, e, *at(p));
    }
    const size_t rowbase = (size_t)b * gridDim.x * S;
    __hip_atomic_store(etag + rowbase + (size_t)blk * S + tid, ((unsigned long long)tag << 32) | __float_as_uint(e),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // 2: the state that enters this block (every block in front of it is a full one)
    const double ad = (double)a;
    const float ap_full = (float)pow(ad, (double)LSQ_TB);
    float h = h0[(size_t)b * S + tid];
    bool timed_out = false;
    for (int j0 = 0; j0 < blk; j0 += LSQ_LOOK) {
      unsigned long long wv[LSQ_LOOK];
      int spins = 0;
      bool ok;
      do {
        ok = true;
#pragma unroll
        for (int i = 0; i < LSQ_LOOK; ++i) {
          const int j = min(j0 + i, blk - 1);
          wv[i] = __hip_atomic_load(etag + rowbase + (size_t)j * S + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int i = 0; i < LSQ_LOOK; ++i) ok = ok && (unsigned)(wv[i] >> 32) == tag;
        if (!ok) __builtin_amdgcn_s_sleep(4);
      } while (!ok && ++spins < LSQ_SPIN_LIMIT);
      timed_out = timed_out || !ok;
#pragma unroll
      for (int i = 0; i < LSQ_LOOK; ++i)
        if (j0 + i < blk) h = fmaf(ap_full, h, __uint_as_float((unsigned)wv[i]));
    }
    if (timed_out) atomicOr(status, 1u);
    if (blk == (int)gridDim.x - 1) {
      const float ap = nvalid == LSQ_TB ? ap_full : (float)pow(ad, (double)nvalid);
      hnew[(size_t)b * S + tid] = fmaf(ap, h, e);
    }
    // 3: the true states of the block's positions
    int p = 0;
    for (; p + 8 <= nvalid; p += 8) {
      float u[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) u[i] = *at(p + i);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        h = fmaf(a, h, u[i]);
        *at(p + i) = h;
      }
    }
    for (; p < nvalid; ++p) {
      h = fmaf(a, h, *at(p));
      *at(p) = h;
    }
  }
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

// clears the published states of the call about to start
__global__ void __launch_bounds__(256) lds_seq_clear_kernel(unsigned long long* __restrict__ etag, size_t n, unsigned* __restrict__ status) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) etag[i] = 0ull;
  if (blockIdx.x == 0 && threadIdx.x == 0) *status = 0u;
}
// the state behind the sequence replaces the caller's h (every block has read h by the time this launch starts)
__global__ void __launch_bounds__(256) lds_seq_finish_kernel(float* __restrict__ h, const float* __restrict__ hnew, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) h[i] = hnew[i];
}

}  // namespace

// workspace: 64 floats of header (status word), the published block states (nblk * Bt * S 64-bit words), the new h
extern "C" size_t fstu_lds_sequence_ws_floats(int T, int Bt, int S) {
  if (T < 0 || Bt < 1 || S < 1) return 0;
  const size_t nblk = (size_t)(T + LSQ_TB - 1) / LSQ_TB;
  return 64 + (2 * nblk + 1) * (size_t)Bt * S;
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
  unsigned* status = (unsigned*)ws;
  unsigned long long* etag = (unsigned long long*)(ws + 64);
  float* hnew = ws + 64 + 2 * (size_t)nblk * BtS;
  const size_t shm = (size_t)LSQ_TB * S * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(nblk, Bt);
  const size_t nwords = (size_t)nblk * BtS;
  unsigned cgrid = (unsigned)((nwords + 255) / 256);
  if (cgrid > 1024u) cgrid = 1024u;
#define LSQ_RUN(NTV)                                                                                                      \
  do {                                                                                                                    \
    static const hipError_t e1 = hipFuncSetAttribute((const void*)lds_seq_kernel<NTV>,                                    \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);            \
    if (e1 != hipSuccess) {                                                                                               \
      fstu_set_error("fstu_lds_sequence: hipFuncSetAttribute: %s", hipGetErrorString(e1));                                \
      return (int)e1;                                                                                                     \
    }                                                                                                                     \
    hipLaunchKernelGGL(lds_seq_clear_kernel, dim3(cgrid), dim3(256), 0, s, etag, nwords, status);                         \
    hipLaunchKernelGGL((lds_seq_kernel<NTV>), grid, dim3(256), shm, s, (const bf16_t*)x, A, (const bf16_t*)BmT,           \
                       (const bf16_t*)CmT, (bf16_t*)y, (const float*)h, hnew, etag, status, 1u, T, Bt, d_in, S, d_out);   \
    hipLaunchKernelGGL(lds_seq_finish_kernel, dim3((unsigned)((BtS + 255) / 256)), dim3(256), 0, s, h, (const float*)hnew, \
                       (int)BtS);                                                                                         \
  } while (0)
  if (S <= 64) LSQ_RUN(4);
  else if (S <= 160) LSQ_RUN(10);
  else LSQ_RUN(16);
#undef LSQ_RUN
  FSTU_CHECK_LAUNCH("fstu_lds_sequence");
  return FSTU_OK;
}

// 0, or 1 when a wait of the last fstu_lds_sequence call on this workspace ran out (synchronous read of the status word)
extern "C" int fstu_lds_sequence_status(const float* ws, int* err_out) {
  FSTU_REQUIRE(ws && err_out, FSTU_ENULL, "fstu_lds_sequence_status: null pointer");
  unsigned v = 0;
  hipError_t e = hipMemcpy(&v, ws, sizeof(v), hipMemcpyDeviceToHost);
  if (e != hipSuccess) { fstu_set_error("fstu_lds_sequence_status: %s", hipGetErrorString(e)); return (int)e; }
  *err_out = (int)v;
  return FSTU_OK;
}
