// Decode-step GEMVs over PACKED bf16 weights, with the residual add + RMSNorm of
// the producer side fused in as a prologue and the split-K reduction fused in as
// an in-kernel fix-up.
//
// Packed layout (built once on the host side from the (N,K) row-major weight):
//   Wp[tile][kstep][lane][8]   tile = n/16, kstep = k/32, lane = 16*g + r,
//   element e of lane (r,g) is W[16*tile + r][32*kstep + 8*g + e]
// i.e. exactly the A-operand fragment of v_mfma_f32_16x16x32_bf16, so one wave
// load instruction (64 lanes x 16 B) reads 1 KB of contiguous memory and a wave
// that walks a K range streams one contiguous block.  Rows beyond N are zero.
//
// Workgroup = 4 waves = 4 K quarters of a run of consecutive 16-feature tiles
// (quarters reduced through LDS in fixed order; the next tile's weights are in
// flight while the current tile is reduced and stored).  Activations are the MFMA B operand: either read from global
// memory, or produced by the prologue into LDS:
//   x_new = T(res_in + delta);  h = T(x_new * rsqrt(mean(x_new^2)+eps) * w)
// (every workgroup recomputes it from the 12-24 KB of inputs; workgroup 0 also
// writes x_new to res_out).  The weight loads of the first K steps are issued
// before the prologue so that HBM latency overlaps it.
#include "fstu_common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

enum { GV_PLAIN = 0, GV_GLU = 1, GV_FIXUP = 2, GV_ARGMAX = 3 };
#define GV_SLOTS 64

__device__ __forceinline__ bf16x8_t gv_as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }

template <int MODE, bool PRO>
__global__ void __launch_bounds__(256)
gemv_packed_kernel(fstu_gemv_args a, int kw /*k per wave*/, int hs_ld /*LDS row stride in elements*/,
                   int tpw /*consecutive tiles per workgroup*/, int ntiles) {
  constexpr int U = 6;  // k steps (32 wide) per load batch
  constexpr int REDF = 4 * 64 * 4 * ((MODE == GV_GLU) ? 2 : 1);   // floats of one reduction buffer
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = (float*)smem;                                        // two reduction buffers (alternating tiles)
  bf16_t* hs = (bf16_t*)(smem + 2 * REDF * sizeof(float));          // rows x hs_ld (PRO only)
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int ksteps_total = a.K >> 5;
  const int ksw = kw >> 5;                                          // k steps per wave
  const int ks0 = (blockIdx.y * 4 + w) * ksw;                       // first k step of this wave
  const int tile0 = blockIdx.x * tpw;
  const int tile1 = min(ntiles, tile0 + tpw);
  const bool xrow = r < a.rows;
  const uint4* wbase = (const uint4*)a.Wp + (size_t)ks0 * 64 + lane;
  const uint4* wbase2 = (MODE == GV_GLU) ? (const uint4*)a.Wp2 + (size_t)ks0 * 64 + lane : nullptr;
  const size_t tile_stride = (size_t)ksteps_total * 64;

  // weights of the first tile's first batch: in flight while the prologue runs
  uint4 wa[U], wb[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (u < ksw) {
      wa[u] = wbase[(size_t)tile0 * tile_stride + (size_t)u * 64];
      if (MODE == GV_GLU) wb[u] = wbase2[(size_t)tile0 * tile_stride + (size_t)u * 64];
    }
  }

  if (PRO) {
    // norm weights of this lane's column chunks: fetched now so that their latency hides behind the first barrier
    const bf16_t* nw = (const bf16_t*)a.norm_w;
    uint4 nwv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = lane * 8 + k * 512;
      nwv[k] = (c < a.K) ? *(const uint4*)(nw + c) : make_uint4(0, 0, 0, 0);
    }
    // ---- x_new = res_in + delta -> LDS (and res_out), 8 elements per thread and iteration
    const int nchunk = a.K >> 3;
    const int total = a.rows * nchunk;
    const bf16_t* xin = (const bf16_t*)a.res_in;
    const bf16_t* dl = (const bf16_t*)a.delta;
    for (int q = threadIdx.x; q < total; q += 256) {
      const int row = q / nchunk, c = (q - row * nchunk) << 3;
      uint4 xv = *(const uint4*)(xin + (size_t)row * a.K + c);
      if (dl) {
        uint4 dv = *(const uint4*)(dl + (size_t)row * a.K + c);
        unsigned xw[4] = {xv.x, xv.y, xv.z, xv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo = __uint_as_float(xw[i] << 16) + __uint_as_float(dw[i] << 16);
          float hi = __uint_as_float(xw[i] & 0xffff0000u) + __uint_as_float(dw[i] & 0xffff0000u);
          xw[i] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
        }
        xv = make_uint4(xw[0], xw[1], xw[2], xw[3]);
        if (blockIdx.x == 0 && blockIdx.y == 0 && a.res_out) *(uint4*)((bf16_t*)a.res_out + (size_t)row * a.K + c) = xv;
      }
      *(uint4*)(hs + (size_t)row * hs_ld + c) = xv;
    }
    __syncthreads();
    // ---- one wave per row: statistics in a fixed order, normalise in place (16-byte LDS accesses)
    for (int row = w; row < a.rows; row += 4) {
      bf16_t* hr = hs + (size_t)row * hs_ld;
      float ss = 0.f;
      for (int c = lane * 8; c < a.K; c += 512) {
        uint4 v = *(const uint4*)(hr + c);
        unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo = __uint_as_float(vw[i] << 16), hi = __uint_as_float(vw[i] & 0xffff0000u);
          ss = fmaf(lo, lo, ss);
          ss = fmaf(hi, hi, ss);
        }
      }
      ss = wave_sum(ss);
      const float rstd = rsqrtf(ss / (float)a.K + a.eps);
      auto scale_chunk = [&](int c, uint4 wv) {
        uint4 v = *(const uint4*)(hr + c);
        unsigned vw[4] = {v.x, v.y, v.z, v.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo = (__uint_as_float(vw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16);
          float hi = (__uint_as_float(vw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u);
          vw[i] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
        }
        *(uint4*)(hr + c) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
      };
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int c = lane * 8 + k * 512;
        if (c < a.K) scale_chunk(c, nwv[k]);
      }
      for (int c = lane * 8 + 2048; c < a.K; c += 512) scale_chunk(c, *(const uint4*)(nw + c));
    }
    __syncthreads();
  }

  const bf16_t* xg = PRO ? nullptr : (const bf16_t*)a.x + (size_t)(xrow ? r : 0) * a.ldx + ks0 * 32 + g * 8;
  const bf16_t* xl = PRO ? hs + (size_t)(xrow ? r : 0) * hs_ld + ks0 * 32 + g * 8 : nullptr;

  for (int tile = tile0; tile < tile1; ++tile) {
    floatx4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    const uint4* wp = wbase + (size_t)tile * tile_stride;
    const uint4* wp2 = (MODE == GV_GLU) ? wbase2 + (size_t)tile * tile_stride : nullptr;
    for (int i0 = 0; i0 < ksw; i0 += U) {
      uint4 xa[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + u < ksw) {
          if (!xrow) xa[u] = make_uint4(0, 0, 0, 0);
          else if (PRO) xa[u] = *(const uint4*)(xl + (size_t)(i0 + u) * 32);
          else xa[u] = *(const uint4*)(xg + (size_t)(i0 + u) * 32);
        }
      }
      uint4 ca[U], cb[U];
#pragma unroll
      for (int u = 0; u < U; ++u) { ca[u] = wa[u]; if (MODE == GV_GLU) cb[u] = wb[u]; }
      // next batch of weights (same tile, or the first batch of the next tile) goes in flight before the MFMAs
      {
        const bool more = i0 + U < ksw;
        const bool next_tile = !more && (tile + 1 < tile1);
        const uint4* np = more ? wp + (size_t)(i0 + U) * 64 : wp + tile_stride;
        const uint4* np2 = (MODE == GV_GLU) ? (more ? wp2 + (size_t)(i0 + U) * 64 : wp2 + tile_stride) : nullptr;
        const int lim = more ? ksw - (i0 + U) : (next_tile ? ksw : 0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u < lim) {
            wa[u] = np[(size_t)u * 64];
            if (MODE == GV_GLU) wb[u] = np2[(size_t)u * 64];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + u < ksw) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv_as_bf16x8(ca[u]), gv_as_bf16x8(xa[u]), acc, 0, 0, 0);
          if (MODE == GV_GLU)
            acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv_as_bf16x8(cb[u]), gv_as_bf16x8(xa[u]), acc2, 0, 0, 0);
        }
      }
    }

    // ---- reduce the 4 K quarters in fixed order (buffers alternate between tiles: one barrier per tile)
    float* rbuf = red + (size_t)((tile - tile0) & 1) * REDF;
    {
      float* mine = rbuf + (size_t)(w * 64 + lane) * 4;
      constexpr int GLU_OFF = 4 * 64 * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mine[i] = acc[i];
        if (MODE == GV_GLU) mine[GLU_OFF + i] = acc2[i];
      }
      __syncthreads();
      if (w != 0) continue;
#pragma unroll
      for (int s = 1; s < 4; ++s) {
        const float* o = rbuf + (size_t)(s * 64 + lane) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[i] += o[i];
          if (MODE == GV_GLU) acc2[i] += o[GLU_OFF + i];
        }
      }
    }

    if (MODE == GV_FIXUP && gridDim.y > 1) {
      // split-K across workgroups: publish this partial tile, the last arriver adds all of them in slice order
      const int GS = gridDim.y;
      float* slot = a.partial_ws + (((size_t)blockIdx.y * ntiles + tile) * 64 + lane) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) __hip_atomic_store(slot + i, acc[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_s_waitcnt(0);   // the partial has reached the coherence point before the ticket is taken
      unsigned old = 0;
      if (lane == 0) old = __hip_atomic_fetch_add(a.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      old = __shfl(old, 0, FSTU_WAVE);
      if (old != (unsigned)(GS - 1)) continue;
      acc = (floatx4_t){0.f, 0.f, 0.f, 0.f};
      for (int s0 = 0; s0 < GS; s0 += 8) {
        float v[8][4];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float* p = a.partial_ws + (((size_t)(s0 + k) * ntiles + tile) * 64 + lane) * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            v[k][i] = (s0 + k < GS) ? __hip_atomic_load(p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += v[k][i];
      }
      if (lane == 0) __hip_atomic_store(a.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if (MODE == GV_ARGMAX) {
      unsigned long long key = 0ull;
      if (xrow) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int f = tile * 16 + g * 4 + i;
          if (f < a.N) {
            float l = DT<bf16_t>::rnd(acc[i]);
            if (a.temperature != 1.0f) l = DT<bf16_t>::rnd(l / a.temperature);
            l = DT<bf16_t>::rnd(fminf(fmaxf(l, -1e4f), 1e4f));
            unsigned u = __float_as_uint(l);
            u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
            unsigned long long k = ((unsigned long long)u << 32) | (unsigned long long)(0xffffffffu - (unsigned)f);
            key = k > key ? k : key;
          }
        }
      }
      unsigned long long o = __shfl_xor(key, 16, FSTU_WAVE);
      key = o > key ? o : key;
      o = __shfl_xor(key, 32, FSTU_WAVE);
      key = o > key ? o : key;
      if (g == 0 && xrow && key != 0ull)
        atomicMax((unsigned long long*)a.best_ws + (size_t)r * GV_SLOTS + (tile & (GV_SLOTS - 1)), key);
    }

    // D layout: lane holds features 4*g+i of batch row r
    if (xrow) {
      bf16_t* yr = (bf16_t*)a.y + (size_t)r * a.ldy;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int f = tile * 16 + g * 4 + i;
        if (f >= a.N) continue;
        if (MODE == GV_GLU) {
          float ge = DT<bf16_t>::rnd(gelu_tanh_f32(DT<bf16_t>::rnd(acc[i])));
          yr[f] = f32_to_bf16(ge * DT<bf16_t>::rnd(acc2[i]));
        } else {
          yr[f] = f32_to_bf16(acc[i]);
        }
      }
    }
  }
}

__global__ void __launch_bounds__(1024)
gv_argmax_finish_kernel(unsigned long long* best, int64_t* tok_out, int64_t stride, int rows, int* dyn, int advance) {
  // one workgroup, one wave per row: max over the slots, then clear them; optionally bump the step counters
  const int b = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = dyn ? dyn[0] : 0;
  __syncthreads();
  if (threadIdx.x == 0 && dyn && advance) { dyn[0] = pos + 1; dyn[1] += 1; }
  if (b >= rows) return;
  unsigned long long k = best[(size_t)b * GV_SLOTS + lane];
  best[(size_t)b * GV_SLOTS + lane] = 0ull;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    unsigned long long t = __shfl_xor(k, o, FSTU_WAVE);
    k = t > k ? t : k;
  }
  if (lane == 0) tok_out[(size_t)b * stride + pos] = (int64_t)(0xffffffffu - (unsigned)(k & 0xffffffffull));
}

static int g_target_wgs = 65535;   // tuning knob: workgroups a GEMV launch aims for

extern "C" int fstu_set_gemv_target_workgroups(int n) {
  FSTU_REQUIRE(n >= 1 && n <= 65535, FSTU_EARG, "fstu_set_gemv_target_workgroups: %d", n);
  g_target_wgs = n;
  return FSTU_OK;
}

template <int MODE>
static void gv_launch(const fstu_gemv_args& a, bool pro, dim3 grid, size_t shm, int kw, int hs_ld, int tpw, int ntiles,
                      hipStream_t s) {
  if (pro) hipLaunchKernelGGL((gemv_packed_kernel<MODE, true>), grid, dim3(256), shm, s, a, kw, hs_ld, tpw, ntiles);
  else hipLaunchKernelGGL((gemv_packed_kernel<MODE, false>), grid, dim3(256), shm, s, a, kw, hs_ld, tpw, ntiles);
}

int fstu_gemv_packed_dyn(const fstu_gemv_args* ap, int* dyn, int advance, void* stream) {
  FSTU_REQUIRE(ap, FSTU_ENULL, "fstu_gemv_packed: null argument block");
  const fstu_gemv_args& a = *ap;
  FSTU_REQUIRE(a.mode >= GV_PLAIN && a.mode <= GV_ARGMAX, FSTU_EARG, "fstu_gemv_packed: mode %d", a.mode);
  FSTU_REQUIRE(a.Wp && a.y, FSTU_ENULL, "fstu_gemv_packed: null weight or output");
  FSTU_REQUIRE(a.rows >= 1 && a.rows <= FSTU_MAX_DECODE_ROWS && a.N >= 1, FSTU_ESHAPE, "fstu_gemv_packed: rows=%d N=%d", a.rows, a.N);
  const int gs = (a.mode == GV_FIXUP) ? (a.ksplit > 0 ? a.ksplit : 1) : 1;
  FSTU_REQUIRE(a.K >= 128 && a.K % (128 * gs) == 0, FSTU_ESHAPE, "fstu_gemv_packed: K=%d must be a multiple of %d", a.K, 128 * gs);
  FSTU_REQUIRE(a.ldy >= a.N, FSTU_ESHAPE, "fstu_gemv_packed: ldy=%d < N=%d", a.ldy, a.N);
  FSTU_REQUIRE(fstu_aligned(a.Wp, 16) && fstu_aligned(a.Wp2, 16), FSTU_EALIGN, "fstu_gemv_packed: packed weights must be 16-byte aligned");
  const bool pro = a.norm_w != nullptr;
  size_t shm = (a.mode == GV_GLU) ? 16384 : 8192;   // two reduction buffers
  int hs_ld = 0;
  if (pro) {
    FSTU_REQUIRE(a.res_in, FSTU_ENULL, "fstu_gemv_packed: norm_w given without res_in");
    FSTU_REQUIRE(a.mode != GV_FIXUP, FSTU_EARG, "fstu_gemv_packed: the prologue is not available with split-K");
    FSTU_REQUIRE(fstu_aligned(a.res_in, 16) && fstu_aligned(a.delta, 16) && fstu_aligned(a.res_out, 16), FSTU_EALIGN,
                 "fstu_gemv_packed: residual pointers must be 16-byte aligned");
    hs_ld = a.K + 8;
    shm += (size_t)a.rows * hs_ld * 2;
    FSTU_REQUIRE(shm <= 64 * 1024, FSTU_ESHAPE, "fstu_gemv_packed: rows*K too large for the fused prologue (%zu bytes of LDS)", shm);
  } else {
    FSTU_REQUIRE(a.x && a.ldx >= a.K && a.ldx % 8 == 0 && fstu_aligned(a.x, 16), FSTU_EARG, "fstu_gemv_packed: bad activation pointer/stride");
  }
  if (a.mode == GV_GLU) FSTU_REQUIRE(a.Wp2, FSTU_ENULL, "fstu_gemv_packed: GLU needs the second packed weight");
  if (a.mode == GV_FIXUP && gs > 1) FSTU_REQUIRE(a.partial_ws && a.counters, FSTU_ENULL, "fstu_gemv_packed: split-K needs partial_ws and counters");
  if (a.mode == GV_ARGMAX) FSTU_REQUIRE(a.best_ws && a.tok_out && a.tok_stride >= 1 && a.temperature > 0.f, FSTU_EARG, "fstu_gemv_packed: greedy pick needs best_ws, tok_out, temperature>0");
  const int ntiles = (a.N + 15) / 16;
  const int kw = a.K / (4 * gs);
  // consecutive tiles per workgroup: about `g_target_wgs` workgroups in flight, so the prologue is paid once per CU
  int tpw = (ntiles * gs + g_target_wgs - 1) / g_target_wgs;
  if (tpw < 1) tpw = 1;
  dim3 grid((ntiles + tpw - 1) / tpw, gs);
  hipStream_t s = (hipStream_t)stream;
  switch (a.mode) {
    case GV_PLAIN: gv_launch<GV_PLAIN>(a, pro, grid, shm, kw, hs_ld, tpw, ntiles, s); break;
    case GV_GLU: gv_launch<GV_GLU>(a, pro, grid, shm, kw, hs_ld, tpw, ntiles, s); break;
    case GV_FIXUP: gv_launch<GV_FIXUP>(a, pro, grid, shm, kw, hs_ld, tpw, ntiles, s); break;
    default: gv_launch<GV_ARGMAX>(a, pro, grid, shm, kw, hs_ld, tpw, ntiles, s); break;
  }
  if (a.mode == GV_ARGMAX)
    hipLaunchKernelGGL(gv_argmax_finish_kernel, dim3(1), dim3(a.rows * 64), 0, s, (unsigned long long*)a.best_ws, a.tok_out,
                       a.tok_stride, a.rows, dyn, advance);
  FSTU_CHECK_LAUNCH("fstu_gemv_packed");
  return FSTU_OK;
}

extern "C" int fstu_gemv_packed(const fstu_gemv_args* a, void* stream) { return fstu_gemv_packed_dyn(a, nullptr, 0, stream); }

// ---------------------------------------------------------------- packing
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
