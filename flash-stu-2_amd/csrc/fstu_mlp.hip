// Decode-step projections of the MLP sub-layer over packed bf16 weights (layout of fstu_pack_rows), one workgroup per
// CU with equal bytes each: the gate/up projection with the GLU epilogue (and the QKV / plain projections on the same
// launch), optionally with the sub-layer's residual add + RMSNorm as its prologue, and the split-K down projection
// (flash_stu/modules/swiglu.py:22-29, flash_stu/layers/stu_layer.py:93-96, flash_stu/layers/attention_layer.py:59-62).
#include <type_traits>
#include "fstu_common.h"
#include "fstu_prologue.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }


// Raw buffer loads: a lane whose byte offset lies beyond the descriptor's range reads zeros without a branch, so
// every load of the kernel sits in straight-line code and the compiler's vmcnt bookkeeping stays exact (the
// activations, issued first, can be consumed while the weight loads issued after them are still in flight).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
#define MLP_OOB 0xfffffff0u
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, p ? (unsigned)bytes : 0u, 0x00020000);
}
__device__ __forceinline__ uint4 buf_load16(rsrc_t rs, unsigned off) {
  u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
// the same for data read exactly once (weights): non-temporal, so that the stream does not push the activations, the
// norm weights and the kernels' own code out of the L2
#ifndef FSTU_WEIGHT_AUX
#define FSTU_WEIGHT_AUX 2
#endif
__device__ __forceinline__ uint4 buf_load16_stream(rsrc_t rs, unsigned off) {
  u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, FSTU_WEIGHT_AUX);
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ u64 pack4_bf16(const float* v) {
  return (u64)pack2_bf16(v[0], v[1]) | ((u64)pack2_bf16(v[2], v[3]) << 32);
}

// sum over each aligned group of 32 lanes, returned in every lane of the group (four DPP steps inside a row of 16
// lanes, one swizzle across the two rows)
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float half_wave_sum(float v) {
  v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);   // row_half_mirror
  v += dpp_f32<0x140>(v);   // row_mirror
  v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));   // lane ^ 16
  return v;
}

// tanh-approximated GELU with tanh(t) = 1 - 2 / (exp(2t) + 1) on the hardware exp and reciprocal: absolute error of
// 1 + tanh about 1e-7, far below the bf16 rounding that follows
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  const float e = __builtin_amdgcn_exp2f(2.8853900817779268f * inner);   // exp(2 inner)
  const float th = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
  return 0.5f * x * (1.0f + th);
}

// rows of `src` (LDS, bf16, stride ld) -> T((v * rstd) * w) into dst (stride ld_dst); wave per row.
// nwv holds the norm weights of this lane's first four column chunks (c = lane*8 + k*512), loaded early.
__device__ __forceinline__ void norm_rows(const bf16_t* src, int ld, bf16_t* dst, int ld_dst, const bf16_t* __restrict__ nw,
                                          const uint4 (&nwv)[4], int rows, int d, float eps, int w, int lane) {
  for (int row = w; row < rows; row += 8) {
    const bf16_t* sr = src + (size_t)row * ld;
    float ss = 0.f;
    for (int c = lane * 8; c < d; c += 512) {
      uint4 v = *(const uint4*)(sr + c);
      unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float lo = __uint_as_float(vw[i] << 16), hi = __uint_as_float(vw[i] & 0xffff0000u);
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
      }
    }
    ss = wave_sum(ss);
    const float rstd = rsqrtf(ss / (float)d + eps);
    auto scale_chunk = [&](int c, uint4 wv) {
      uint4 v = *(const uint4*)(sr + c);
      unsigned vw[4] = {v.x, v.y, v.z, v.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float lo = (__uint_as_float(vw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16);
        float hi = (__uint_as_float(vw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u);
        vw[i] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
      }
      *(uint4*)(dst + (size_t)row * ld_dst + c) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
    };
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = lane * 8 + k * 512;
      if (c < d) scale_chunk(c, nwv[k]);
    }
    for (int c = lane * 8 + 2048; c < d; c += 512) scale_chunk(c, *(const uint4*)(nw + c));
  }
}

__device__ __forceinline__ void load_norm_w(uint4 (&nwv)[4], const bf16_t* __restrict__ nw, int d, int lane) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int c = lane * 8 + k * 512;
    nwv[k] = buf_load16(make_rsrc(nw, (size_t)d * 2), c < d ? (unsigned)c * 2u : MLP_OOB);
  }
}

// ---------------------------------------------------------------- balanced gate/up GEMV (stand-alone launch)
// One workgroup per CU, I/G features each in groups of 8 (equal bytes per CU), every weight fragment of a workgroup in
// flight from the first instruction, the 8 waves split K.
struct GluArgs {
  const bf16_t* h;        // normalised input (rows x ldh); unused with the prologue
  const uint4* wp_gate;
  const uint4* wp_up;
  bf16_t* act;
  int rows, d, I, ldh, ldact, fpw;
  // prologue (PRO): h = rmsnorm(T(x_in + delta)) * norm_w computed by every workgroup; workgroup 0 stores the sum
  // (PRO 2: delta = up to 4 fp32 split-K slices of (rows x d), summed in order and rounded before the add)
  const bf16_t* x_in;
  const void* delta;
  bf16_t* x_out;
  const bf16_t* norm_w;
  float eps;
  int nslices;
  // EPI 2: per-row packed maxima (rows x 64 words, zero on entry) of the logits at this temperature
  unsigned long long* best;
  float temperature;
};

// EPI 0: act = gelu(gate)*up (two matrices);  1: y = x W^T;  2: y = x W^T plus, per row, the packed maxima
// (value key of the logit at `temperature`, ~index) of 64 subsets of the features, into `best` as 64-bit words
// (the tied head in front of the greedy pick or of the spread sampler)
// (arguments passed one by one so that the command processor can preload the leading ones into SGPRs)
// NB = 2 (no prologue): rows 16..31 are a second B tile of the same weight fragments, so 17..32 rows read every weight
// once; the partial sums of the two row tiles then lie behind each other in dynamic LDS.
template <int KSA, int PRO, int EPI, int NB = 1>
__global__ void __launch_bounds__(512)
glu_balanced_kernel(const bf16_t* h, const uint4* wp_gate, const uint4* wp_up, bf16_t* act, const bf16_t* x_in,
                    const void* delta, bf16_t* x_out, const bf16_t* norm_w, int rows, int d, int I, int ldh, int ldact,
                    int fpw, float eps, int nslices, unsigned long long* best, float temperature) {
  GluArgs a;
  a.h = h; a.wp_gate = wp_gate; a.wp_up = wp_up; a.act = act; a.rows = rows; a.d = d; a.I = I; a.ldh = ldh; a.ldact = ldact;
  a.fpw = fpw; a.x_in = x_in; a.delta = delta; a.x_out = x_out; a.norm_w = norm_w; a.eps = eps; a.nslices = nslices;
  a.best = best; a.temperature = temperature;
  constexpr bool GLU = EPI == 0;
  constexpr int DA = KSA <= 3 ? 4 : (KSA == 4 ? 3 : 2);
  constexpr int NXC = 4;
  static_assert(PRO == 3 ? NB == 2 : (NB == 1 || PRO == 0), "two row tiles: no prologue, or the in-register one (PRO 3)");
  constexpr int RED = DA * 8 * 512;                           // partial sums of one row tile
  __shared__ float red_one[NB == 1 ? RED : 1];
  extern __shared__ __align__(16) unsigned char glu_smem[];   // PRO: h rows (rows x (d+8)) bf16; NB 2: the partial sums
  float* red = NB == 1 ? red_one : (float*)glu_smem;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int wgi = blockIdx.x;
  const bool xrow = r < a.rows;
  uint4 xa[KSA];
  uint4 xa2[NB == 2 ? KSA : 1];                               // B fragments of rows 16..31
  const int nchunk = a.d >> 3, total = a.rows * nchunk;
  // weight addressing
  // Features are dealt out in groups of 8 (a.fpw == 0): with the packed layout a group of 8 rows is one whole 128-byte
  // line per k group, so no line is shared with (and fetched again by) the neighbouring workgroup on another XCD.
  int f0, f1;
  if (a.fpw > 0) {
    f0 = wgi * a.fpw;
    f1 = min(a.I, f0 + a.fpw);
  } else {
    const long long ngr = (a.I + 7) >> 3;
    f0 = (int)(ngr * wgi / gridDim.x) * 8;
    f1 = min(a.I, (int)(ngr * (wgi + 1) / gridDim.x) * 8);
  }
  const int ta0 = f0 >> 4, ta1 = (f1 > f0) ? ((f1 + 15) >> 4) : ta0;
  const size_t tsa = (size_t)(a.d >> 5) * 64;
  const size_t wa_bytes = (size_t)((a.I + 15) >> 4) * tsa * 16;
  const rsrc_t rg = make_rsrc(a.wp_gate, wa_bytes), ru = make_rsrc(a.wp_up, wa_bytes);
  const unsigned abase = ((unsigned)(w * KSA) * 64 + lane) * 16u;
  uint4 wa[DA][KSA], wb[DA][KSA];
  auto load_a = [&](int j, int tile) {
    const int f = tile * 16 + r;
    const bool ok = tile < ta1 && f >= f0 && f < f1;
#pragma unroll
    for (int u = 0; u < KSA; ++u) {
      const unsigned off = ok ? abase + ((unsigned)tile * (unsigned)tsa + (unsigned)u * 64u) * 16u : MLP_OOB;
      wa[j][u] = buf_load16_stream(rg, off);
      if (GLU) wb[j][u] = buf_load16_stream(ru, off);
    }
  };
  // a tile beyond the workgroup's range is skipped by a uniform branch: a load of nothing still costs its address cycles
  auto load_first = [&]() {
#pragma unroll
    for (int j = 0; j < DA; ++j)
      if (ta0 + j < ta1) load_a(j, ta0 + j);
  };

  if constexpr (PRO == 0) {
    // activations first (they are consumed first), then the weights
    const rsrc_t rh = make_rsrc(a.h, ((size_t)(a.rows - 1) * a.ldh + a.d) * 2);
    const unsigned hoff = ((unsigned)(xrow ? r : 0) * (unsigned)a.ldh + (unsigned)(w * KSA) * 32u + (unsigned)g * 8u) * 2u;
#pragma unroll
    for (int u = 0; u < KSA; ++u) xa[u] = buf_load16(rh, xrow ? hoff + (unsigned)u * 64u : MLP_OOB);
    if constexpr (NB == 2) {
      const bool xrow2 = 16 + r < a.rows;
#pragma unroll
      for (int u = 0; u < KSA; ++u) xa2[u] = buf_load16(rh, xrow2 ? hoff + (unsigned)(16 * a.ldh) * 2u + (unsigned)u * 64u : MLP_OOB);
    }
    load_first();
  } else if constexpr (PRO == 3) {
    // Two row tiles (17..32 dense rows of stride d), x_in = the residual stream with the sub-layer's output already
    // added: h = T((x * rstd) * w) is formed in the B fragments themselves.  A row's sum of squares goes over the
    // four lane groups by shuffles and over the 8 waves (which split K) through LDS, as do the norm weights (kept in
    // registers next to both row tiles and the weight fragments they would spill).  All of it happens while the
    // weights, requested right behind the activations, are on their way.
    __shared__ float ss_part[8][32];
    __shared__ __align__(16) unsigned nw_s[128 * KSA];
    constexpr int NWD = (KSA + 3) / 4;
    unsigned nwt[NWD];
    const rsrc_t rxi = make_rsrc(a.x_in, (size_t)a.rows * a.d * 2), rnw = make_rsrc(a.norm_w, (size_t)a.d * 2);
    const unsigned koff = ((unsigned)(w * KSA) * 32u + (unsigned)g * 8u) * 2u;
    const unsigned o1 = (unsigned)r * (unsigned)a.d * 2u + koff, o2 = o1 + 16u * (unsigned)a.d * 2u;
    const bool xrow2 = 16 + r < a.rows;
#pragma unroll
    for (int u = 0; u < KSA; ++u) xa[u] = buf_load16(rxi, xrow ? o1 + (unsigned)u * 64u : MLP_OOB);
#pragma unroll
    for (int u = 0; u < KSA; ++u) xa2[u] = buf_load16(rxi, xrow2 ? o2 + (unsigned)u * 64u : MLP_OOB);
#pragma unroll
    for (int k = 0; k < NWD; ++k) {
      const unsigned i = threadIdx.x + k * 512u;
      nwt[k] = __builtin_amdgcn_raw_buffer_load_b32(rnw, i < 128u * KSA ? i * 4u : MLP_OOB, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);   // the activations' requests stay in front of the weights'
    // One tile of weights (16 KB per wave) goes out behind them, the others after the rows are scaled: with every
    // tile of every workgroup queued at once the activations come back late (38.3 against 36.5 us for the launch
    // at 2048 x 24576).
    load_a(0, ta0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    auto squares = [](uint4 v, float& ss) {
      const unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(vw[i] << 16), hi = __uint_as_float(vw[i] & 0xffff0000u);
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
      }
    };
    float ss1 = 0.f, ss2 = 0.f;
#pragma unroll
    for (int u = 0; u < KSA; ++u) {
      squares(xa[u], ss1);
      squares(xa2[u], ss2);
    }
    // the rows stay packed until they are scaled: without this the unpacked values of the squares above (twice the
    // registers) are kept for the scaling below and spill
#pragma unroll
    for (int u = 0; u < KSA; ++u) {
      asm volatile("" : "+v"(xa[u].x), "+v"(xa[u].y), "+v"(xa[u].z), "+v"(xa[u].w));
      asm volatile("" : "+v"(xa2[u].x), "+v"(xa2[u].y), "+v"(xa2[u].z), "+v"(xa2[u].w));
    }
    ss1 += __shfl_xor(ss1, 16, 64);
    ss1 += __shfl_xor(ss1, 32, 64);
    ss2 += __shfl_xor(ss2, 16, 64);
    ss2 += __shfl_xor(ss2, 32, 64);
    if (g == 0) { ss_part[w][r] = ss1; ss_part[w][16 + r] = ss2; }
#pragma unroll
    for (int k = 0; k < NWD; ++k) {
      const unsigned i = threadIdx.x + k * 512u;
      if (i < 128u * KSA) nw_s[i] = nwt[k];
    }
    __syncthreads();
    float t1 = 0.f, t2 = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) { t1 += ss_part[s][r]; t2 += ss_part[s][16 + r]; }
    const float rs1 = rsqrtf(t1 / (float)a.d + a.eps), rs2 = rsqrtf(t2 / (float)a.d + a.eps);
    auto scale8 = [](uint4 v, uint4 wv, float rstd) {
      unsigned vw[4] = {v.x, v.y, v.z, v.w};
      const unsigned ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
        vw[i] = pack2_bf16((__uint_as_float(vw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16),
                           (__uint_as_float(vw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u));
      return make_uint4(vw[0], vw[1], vw[2], vw[3]);
    };
#pragma unroll
    for (int u = 0; u < KSA; ++u) {
      const uint4 nwv = *(const uint4*)(nw_s + (w * KSA + u) * 16 + g * 4);
      xa[u] = scale8(xa[u], nwv, rs1);
      xa2[u] = scale8(xa2[u], nwv, rs2);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 1; j < DA; ++j)
      if (ta0 + j < ta1) load_a(j, ta0 + j);
  } else {
    // x' = T(x + delta) (workgroup 0 also stores it), h = T((x' * rstd) * w) into LDS, then this wave's B fragments.
    // The 24 KB of x and delta are requested and consumed BEFORE the weights are requested: they return at
    // idle-memory latency instead of queueing behind every workgroup's weight stream, nothing the norm needs is
    // left behind the weight loads in the load counter, and the second half of the norm runs while the weights
    // arrive.
    bf16_t* hs = (bf16_t*)glu_smem;
    const int ld = a.d + 8;
    auto add_chunk = [&](uint4 x4, uint4 d4, float& ss) {
      unsigned xw[4] = {x4.x, x4.y, x4.z, x4.w}, dw[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xw[i] = pack2_bf16(__uint_as_float(xw[i] << 16) + __uint_as_float(dw[i] << 16),
                           __uint_as_float(xw[i] & 0xffff0000u) + __uint_as_float(dw[i] & 0xffff0000u));
        const float lo = __uint_as_float(xw[i] << 16), hi = __uint_as_float(xw[i] & 0xffff0000u);
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
      }
      return make_uint4(xw[0], xw[1], xw[2], xw[3]);
    };
    // the lean prologue, instantiated for the exact number of chunks per thread so that it is one straight line
    auto lean = [&](auto nxc_tag) {
      constexpr int NX = decltype(nxc_tag)::value;
      typedef NormPrologue<512, NX, PRO == 2 ? 4 : 0> Pro;
      // the activations are requested first; x' and the row statistics are formed as soon as they are there, the
      // scaling runs while the weights arrive
      __shared__ float ss_part[Pro::NPART];
      Pro pro;
      pro.issue(a.x_in, a.delta, a.nslices, a.norm_w, a.rows, a.d);
      __builtin_amdgcn_sched_barrier(0);   // the activations' requests stay in front of the weights'
      // One tile's weights go out right behind the activations, the rest after x' and the row statistics are formed:
      // with every weight request of every workgroup queued at once the 24 KB of activations come back only with the
      // end of the 28 MB (measured: 4.9 us instead of 2 us after the first instruction).  Only the last tile is
      // conditional, so that the norm weights, requested earlier, keep an exact position in the load counter.
      load_a(0, ta0);
      asm volatile("" ::: "memory");   // the loads above are neither sunk below the branches of the reduction
      __builtin_amdgcn_sched_barrier(0);   // nor overtaken by its arithmetic (which waits for the activations)
      pro.reduce(ss_part, wgi == 0 ? a.x_out : nullptr, a.rows, a.d);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 1; j < DA; ++j)
        if (j < DA - 1 || ta0 + j < ta1) load_a(j, ta0 + j);
      __syncthreads();
      pro.scale(ss_part, hs, ld, a.rows, a.d, a.eps);
    };
    constexpr int NXMAX = PRO == 2 ? 2 : NXC;
    if (total <= 512 && (nchunk & 31) == 0) {
      lean(std::integral_constant<int, 1>{});
    } else if (total <= 1024 && (nchunk & 31) == 0) {
      lean(std::integral_constant<int, 2>{});
    } else if (NXMAX >= 4 && total <= 2048 && (nchunk & 31) == 0) {
      lean(std::integral_constant<int, NXMAX>{});
    } else if (PRO == 1) {
      // any other shape: wave per row
      uint4 nwv[4];
      load_norm_w(nwv, a.norm_w, a.d, lane);
      for (int q = threadIdx.x; q < total; q += 512) {
        const int row = q / nchunk, c = (q - row * nchunk) << 3;
        float ss = 0.f;
        uint4 v = *(const uint4*)(a.x_in + (size_t)q * 8);
        if (a.delta) v = add_chunk(v, *(const uint4*)((const bf16_t*)a.delta + (size_t)q * 8), ss);
        *(uint4*)(hs + (size_t)row * ld + c) = v;
        if (wgi == 0 && a.x_out) *(uint4*)(a.x_out + (size_t)q * 8) = v;
      }
      __builtin_amdgcn_sched_barrier(0);
      load_first();
      __syncthreads();
      norm_rows(hs, ld, hs, ld, a.norm_w, nwv, a.rows, a.d, a.eps, w, lane);
    }
    __syncthreads();
    const bf16_t* hl = hs + (size_t)(xrow ? r : 0) * ld + (w * KSA) * 32 + g * 8;
#pragma unroll
    for (int u = 0; u < KSA; ++u) xa[u] = xrow ? *(const uint4*)(hl + u * 32) : make_uint4(0, 0, 0, 0);
  }

  unsigned long long run_key[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) run_key[nb] = 0ull;
  for (int t0 = ta0; t0 < ta1; t0 += DA) {
#pragma unroll
    for (int j = 0; j < DA; ++j) {
      if (t0 + j >= ta1) continue;   // uniform
      floatx4_t acc[NB], acc2[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = acc2[nb] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < KSA; ++u) {
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[j][u]), as_bf16x8(xa[u]), acc[0], 0, 0, 0);
        if (GLU) acc2[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb[j][u]), as_bf16x8(xa[u]), acc2[0], 0, 0, 0);
        if constexpr (NB == 2) {
          acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[j][u]), as_bf16x8(xa2[u]), acc[1], 0, 0, 0);
          if (GLU) acc2[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb[j][u]), as_bf16x8(xa2[u]), acc2[1], 0, 0, 0);
        }
      }
      if (t0 + DA + j < ta1) load_a(j, t0 + DA + j);   // uniform: a load of nothing still costs its address cycles
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float* mine = red + (size_t)nb * RED + (size_t)((j * 8 + w) * 2 * 64 + lane) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          mine[i] = acc[nb][i];
          if (GLU) mine[256 + i] = acc2[nb][i];
        }
      }
    }
    // EPI 1 with x_out: the projection's output joins the residual stream here, x_out = T(x_in + T(y)) (rows of stride
    // ldact in both); the pairs of x_in this wave will need are requested before the barrier
    unsigned resw[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) resw[nb] = 0u;
    if constexpr (EPI == 1 && PRO == 0) {
      if (a.x_out) {
        const int fbp = (t0 + (w >> 1)) * 16 + g * 4 + (w & 1) * 2;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int row = 16 * nb + r;
          const bool okp = (w >> 1) < DA && row < a.rows && fbp >= f0 && fbp + 2 <= f1;
          resw[nb] = okp ? *(const unsigned*)(a.x_in + (size_t)row * a.ldact + fbp) : 0u;
        }
      }
    }
    __syncthreads();
    // reduction over the 8 K slices and the epilogue: wave w takes half a tile (two of a lane's four features)
    if ((w >> 1) < DA && t0 + (w >> 1) < ta1) {
      const int jt = w >> 1, hf = (w & 1) * 2;
      const int tile = t0 + jt;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float sg[2] = {0.f, 0.f}, su[2] = {0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const float* o = red + (size_t)nb * RED + (size_t)((jt * 8 + s) * 2 * 64 + lane) * 4 + hf;
          const float2 pg = *(const float2*)o;
          sg[0] += pg.x;
          sg[1] += pg.y;
          if (GLU) {
            const float2 pu = *(const float2*)(o + 256);
            su[0] += pu.x;
            su[1] += pu.y;
          }
        }
        const int fb = tile * 16 + g * 4 + hf;
        float o[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if (GLU) {
            float ge = DT<bf16_t>::rnd(gelu_tanh_fast(DT<bf16_t>::rnd(sg[i])));
            o[i] = ge * DT<bf16_t>::rnd(su[i]);
          } else {
            o[i] = sg[i];
          }
        }
        // the workgroup's range starts and ends on a multiple of four features, so a pair is inside it or outside it
        const int row = 16 * nb + r;
        const bool grp_ok = row < a.rows && fb >= f0 && fb < f1;
        if constexpr (EPI == 2) {
          // best (value, lowest index) of this lane's features so far; the workgroup's lanes are merged after its
          // last tile
          const float temperature = a.temperature;
          unsigned long long key = 0ull;
          if (grp_ok) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
              if (fb + i < f1) {
                float l = DT<bf16_t>::rnd(o[i]);
                if (temperature != 1.0f) l = DT<bf16_t>::rnd(l / temperature);
                l = DT<bf16_t>::rnd(fminf(fmaxf(l, -1e4f), 1e4f));
                unsigned u = __float_as_uint(l);
                u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                const unsigned long long k = ((unsigned long long)u << 32) | (unsigned long long)(0xffffffffu - (unsigned)(fb + i));
                key = k > key ? k : key;
              }
            }
          }
          run_key[nb] = key > run_key[nb] ? key : run_key[nb];
        }
        if (EPI == 1 && PRO == 0 && a.x_out) {
          // (feature ranges start and end on multiples of 8 and ldact is even here: whole pairs only)
          if (grp_ok) {
            const float y0 = DT<bf16_t>::rnd(o[0]), y1 = DT<bf16_t>::rnd(o[1]);
            *(unsigned*)(a.x_out + (size_t)row * a.ldact + fb) =
                pack2_bf16(__uint_as_float(resw[nb] << 16) + y0, __uint_as_float(resw[nb] & 0xffff0000u) + y1);
          }
        } else if (grp_ok) {
          bf16_t* yr = a.act + (size_t)row * a.ldact + fb;
          if (fb + 2 <= f1 && (a.ldact & 1) == 0) {
            *(unsigned*)yr = pack2_bf16(o[0], o[1]);
          } else {
#pragma unroll
            for (int i = 0; i < 2; ++i)
              if (fb + i < f1) yr[i] = f32_to_bf16(o[i]);
          }
        }
      }
    }
    if (t0 + DA < ta1) __syncthreads();
  }
  if constexpr (EPI == 2) {
    // Per row: the best of the workgroup's whole feature range, then ONE 64-bit atomic max per row and workgroup into
    // slot (workgroup & 63) of the row: the slots stay disjoint subsets of the vocabulary (4 workgroups each on a
    // grid of 256), and the launch issues a few thousand atomics instead of one per row and half tile
    unsigned long long* best = a.best;
    unsigned long long* keys = (unsigned long long*)red;          // 8 waves x NB x 16 rows
    __syncthreads();                                              // the last reduction has read `red`
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      unsigned long long key = run_key[nb];
      unsigned long long ok = __shfl_xor(key, 16, 64);
      key = ok > key ? ok : key;
      ok = __shfl_xor(key, 32, 64);
      key = ok > key ? ok : key;
      if (g == 0) keys[(w * NB + nb) * 16 + r] = key;
    }
    __syncthreads();
    if (threadIdx.x < NB * 16) {
      const int nb = threadIdx.x >> 4, rr = threadIdx.x & 15;
      unsigned long long key = 0ull;
#pragma unroll
      for (int ww = 0; ww < 8; ++ww) {
        const unsigned long long o = keys[(ww * NB + nb) * 16 + rr];
        key = o > key ? o : key;
      }
      const int row = 16 * nb + rr;
      if (row < a.rows && key != 0ull) atomicMax(best + (size_t)row * 64 + (wgi & 63), key);
    }
  }
}

// ---------------------------------------------------------------- balanced split-K down projection (stand-alone launch)
// partial[chunk][row][feature] (fp32 slices, the layout fstu_add_rmsnorm sums): workgroup (tile group, K chunk), every
// weight fragment and the activations of the chunk in flight from the first
// instruction, the 8 waves split the chunk's k steps and are reduced through LDS in wave order.
struct DownSkArgs {
  const bf16_t* act;
  const uint4* wp_down;
  float* partial;      // KS x rows x d
  int rows, d, I, ldact, KS, tpw, tiles_out, kch;
};

// NB = 2: rows 16..31 as a second B tile of the same weight fragments (17..32 rows read every weight once).
template <int KSB, int NB = 1>
__global__ void __launch_bounds__(512)
down_splitk_balanced_kernel(const bf16_t* act, const uint4* wp_down, float* partial, int rows, int d, int I, int ldact, int KS,
                            int tpw, int tiles_out, int kch) {
  const DownSkArgs a{act, wp_down, partial, rows, d, I, ldact, KS, tpw, tiles_out, kch};
  constexpr int DB = KSB <= 3 ? 4 : (KSB == 4 ? 3 : (KSB <= 8 ? 2 : 1));
  constexpr int RED = DB * 8 * 256;                          // partial sums of one row tile
  __shared__ float red[NB * RED];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const bool xrow = r < a.rows;
  const int chunk = blockIdx.x % a.KS, tgrp = blockIdx.x / a.KS;
  const int tb0 = tgrp * a.tpw, tb1 = min(a.tiles_out, tb0 + a.tpw);
  const int ksb0 = w * KSB;
  const int nks = max(0, min(KSB, a.kch - ksb0));
  const size_t tsb = (size_t)(a.I >> 5) * 64;
  // activations of this wave's k steps first, then the weights
  const rsrc_t rx = make_rsrc(a.act, ((size_t)(a.rows - 1) * a.ldact + a.I) * 2);
  const unsigned xbase = ((unsigned)(xrow ? r : 0) * (unsigned)a.ldact + (unsigned)(chunk * a.kch + ksb0) * 32u + (unsigned)g * 8u) * 2u;
  uint4 xb[KSB];
  uint4 xb2[NB == 2 ? KSB : 1];                               // B fragments of rows 16..31
#pragma unroll
  for (int u = 0; u < KSB; ++u) xb[u] = buf_load16(rx, (xrow && u < nks) ? xbase + (unsigned)u * 64u : MLP_OOB);
  if constexpr (NB == 2) {
    const bool xrow2 = 16 + r < a.rows;
#pragma unroll
    for (int u = 0; u < KSB; ++u)
      xb2[u] = buf_load16(rx, (xrow2 && u < nks) ? xbase + (unsigned)(16 * a.ldact) * 2u + (unsigned)u * 64u : MLP_OOB);
  }
  const rsrc_t rdn = make_rsrc(a.wp_down, (size_t)a.tiles_out * tsb * 16);
  const unsigned bbase = ((unsigned)(chunk * a.kch + ksb0) * 64 + lane) * 16u;
  uint4 wd[DB][KSB];
  auto load_b = [&](int j, int tile) {
#pragma unroll
    for (int u = 0; u < KSB; ++u)
      wd[j][u] = buf_load16_stream(rdn, (u < nks && tile < tb1) ? bbase + ((unsigned)tile * (unsigned)tsb + (unsigned)u * 64u) * 16u : MLP_OOB);
  };
  // waves beyond the chunk's k steps and tiles beyond the group's range are skipped by uniform branches: a load of
  // nothing still costs its address cycles
  const bool active = nks > 0;
  const int nact = min(8, (a.kch + KSB - 1) / KSB);
  if (active) {
#pragma unroll
    for (int j = 0; j < DB; ++j)
      if (tb0 + j < tb1) load_b(j, tb0 + j);
  }
  for (int t0 = tb0; t0 < tb1; t0 += DB) {
    if (active) {
#pragma unroll
      for (int j = 0; j < DB; ++j) {
        if (t0 + j >= tb1) continue;
        floatx4_t acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KSB; ++u) {
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wd[j][u]), as_bf16x8(xb[u]), acc[0], 0, 0, 0);
          if constexpr (NB == 2)
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wd[j][u]), as_bf16x8(xb2[u]), acc[1], 0, 0, 0);
        }
        if (t0 + DB + j < tb1) load_b(j, t0 + DB + j);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          float* mine = red + (size_t)nb * RED + (size_t)((j * 8 + w) * 64 + lane) * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[i] = acc[nb][i];
        }
      }
    }
    __syncthreads();
    // reduction over the K slices of the active waves: wave w takes half a tile (two of a lane's four features)
    if ((w >> 1) < DB && t0 + (w >> 1) < tb1) {
      const int jt = w >> 1, hf = (w & 1) * 2;
      const int tile = t0 + jt;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float sd[2] = {0.f, 0.f};
        for (int s = 0; s < nact; ++s) {
          const float2 o = *(const float2*)(red + (size_t)nb * RED + (size_t)((jt * 8 + s) * 64 + lane) * 4 + hf);
          sd[0] += o.x;
          sd[1] += o.y;
        }
        // D layout: features tile*16 + 4g + i of batch row r of the row tile
        const int fb = tile * 16 + 4 * g + hf, row = 16 * nb + r;
        if (row < a.rows && fb < a.d) *(float2*)(a.partial + ((size_t)chunk * a.rows + row) * a.d + fb) = make_float2(sd[0], sd[1]);
      }
    }
    if (t0 + DB < tb1) __syncthreads();
  }
}

int g_cus = 0;
}  // namespace

static int query_cus() {
  if (g_cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return 0;
    g_cus = p.multiProcessorCount;
  }
  return g_cus;
}

extern "C" int fstu_glu_packed_supported(int rows, int d, int I) {
  const int ksa = d / 256;
  return rows >= 1 && rows <= FSTU_MAX_DECODE_ROWS && d % 256 == 0 && (ksa == 1 || ksa == 2 || ksa == 3 || ksa == 4 || ksa == 8) &&
         I >= 16 && (size_t)I * d * 2 < 0xfff00000ull;
}

// 17..32 rows: fstu_glu_packed and fstu_down_packed_splitk take them as two row tiles per weight fragment (the launches
// with a norm prologue do not)
extern "C" int fstu_mlp_packed_rows32_supported(int rows, int d, int I) {
  return rows > FSTU_MAX_DECODE_ROWS && rows <= 2 * FSTU_MAX_DECODE_ROWS && fstu_glu_packed_supported(FSTU_MAX_DECODE_ROWS, d, I) &&
         I % 512 == 0 && (size_t)rows * I * 2 < 0x7ff00000ull;
}

template <int KSA>
static int glu_launch_ksa(GluArgs& a, int pro, int epi, int G, size_t shm, const char* name, hipStream_t s) {
#define GLU_GO(PRO, GLUF)                                                                                        \
  do {                                                                                                           \
    if (shm > 0) {                                                                                               \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(glu_balanced_kernel<KSA, PRO, GLUF>),     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);                  \
      FSTU_REQUIRE(e == hipSuccess, (int)e, "%s: %zu bytes of dynamic LDS refused", name, shm);                  \
    }                                                                                                            \
    hipLaunchKernelGGL((glu_balanced_kernel<KSA, PRO, GLUF>), dim3(G), dim3(512), shm, s, a.h, a.wp_gate, a.wp_up, a.act, a.x_in,    \
                       a.delta, a.x_out, a.norm_w, a.rows, a.d, a.I, a.ldh, a.ldact, a.fpw, a.eps, a.nslices, a.best, a.temperature); \
  } while (0)
  if (a.rows > FSTU_MAX_DECODE_ROWS) {
    // two row tiles: the partial sums of both lie in dynamic LDS
    constexpr int DA = KSA <= 3 ? 4 : (KSA == 4 ? 3 : 2);
    const size_t red2 = (size_t)2 * DA * 8 * 512 * sizeof(float);
    FSTU_REQUIRE(pro == 0 || (pro == 3 && epi != 2), FSTU_ESHAPE, "%s: more than %d rows: no prologue, or the in-register one (not on the head)",
                 name, FSTU_MAX_DECODE_ROWS);
#define GLU_GO2(PRO, EPI)                                                                                                  \
  do {                                                                                                                     \
    static hipError_t attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(glu_balanced_kernel<KSA, PRO, EPI, 2>),  \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)red2);               \
    FSTU_REQUIRE(attr_err == hipSuccess, (int)attr_err, "%s: %zu bytes of dynamic LDS refused", name, red2);               \
    hipLaunchKernelGGL((glu_balanced_kernel<KSA, PRO, EPI, 2>), dim3(G), dim3(512), red2, s, a.h, a.wp_gate, a.wp_up, a.act, \
                       a.x_in, a.delta, a.x_out, a.norm_w, a.rows, a.d, a.I, a.ldh, a.ldact, a.fpw, a.eps, a.nslices, a.best,  \
                       a.temperature);                                                                                      \
  } while (0)
    if (pro == 3 && epi == 0) GLU_GO2(3, 0);
    else if (pro == 3) GLU_GO2(3, 1);
    else if (epi == 0) GLU_GO2(0, 0);
    else if (epi == 2) GLU_GO2(0, 2);
    else GLU_GO2(0, 1);
#undef GLU_GO2
    return FSTU_OK;
  }
  if (pro == 2) GLU_GO(2, 1);
  else if (pro && epi == 0) GLU_GO(1, 0);
  else if (pro) GLU_GO(1, 1);
  else if (epi == 0) GLU_GO(0, 0);
  else if (epi == 2) GLU_GO(0, 2);
  else GLU_GO(0, 1);
#undef GLU_GO
  return FSTU_OK;
}

static int glu_launch(GluArgs& a, int pro, int epi, const char* name, hipStream_t s) {
  int G = query_cus();
  FSTU_REQUIRE(G > 0, FSTU_EARG, "%s: no device", name);
  // Features are dealt out in groups of 8: no 128-byte line is shared between two workgroups (HBM traffic of the
  // gate/up launch 1.00x the algorithmic bytes instead of 1.125x with groups of 4), at the price of workgroups of 32
  // and 40 features instead of 36 each.
  // the head (thousands of tiles, one weight matrix: half the bytes in flight per workgroup of the gated pair) runs two
  // workgroups per compute unit where registers and LDS allow it
  if (epi == 2 && a.rows <= FSTU_MAX_DECODE_ROWS && a.d <= 1024) G *= 2;
  if (G > (a.I + 7) / 8) G = (a.I + 7) / 8;
  // a plain projection narrower than 16 features per CU (QKV at d = 768: 2304 features) gets one whole tile per
  // workgroup rather than half tiles on every CU: every workgroup repeats the norm prologue, and its operands come
  // out of one L2 per XCD
  if (epi != 0 && G > (a.I + 15) / 16) G = (a.I + 15) / 16;
  a.fpw = 0;
  const size_t shm = (pro == 1 || pro == 2) ? (size_t)a.rows * (a.d + 8) * 2 : 0;
  int rc;
  switch (a.d / 256) {
    case 1: rc = glu_launch_ksa<1>(a, pro, epi, G, shm, name, s); break;
    case 2: rc = glu_launch_ksa<2>(a, pro, epi, G, shm, name, s); break;
    case 3: rc = glu_launch_ksa<3>(a, pro, epi, G, shm, name, s); break;
    case 4: rc = glu_launch_ksa<4>(a, pro, epi, G, shm, name, s); break;
    default: rc = glu_launch_ksa<8>(a, pro, epi, G, shm, name, s); break;
  }
  if (rc) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fstu_set_error("%s: launch failed: %s", name, hipGetErrorString(e));
    return (int)e;
  }
  return FSTU_OK;
}

extern "C" int fstu_glu_packed(const void* h, int ldh, const void* wp_gate, const void* wp_up, void* act, int ldact, int rows,
                               int I, int d, void* stream) {
  FSTU_REQUIRE(h && wp_gate && wp_up && act, FSTU_ENULL, "fstu_glu_packed: null pointer");
  FSTU_REQUIRE(fstu_glu_packed_supported(rows, d, I) || fstu_mlp_packed_rows32_supported(rows, d, I), FSTU_ESHAPE,
               "fstu_glu_packed: unsupported shape rows=%d d=%d I=%d", rows, d, I);
  FSTU_REQUIRE(ldh >= d && ldh % 8 == 0 && ldact >= I && ldact % 4 == 0, FSTU_ESHAPE, "fstu_glu_packed: ldh=%d ldact=%d", ldh, ldact);
  FSTU_REQUIRE(fstu_aligned(h, 16) && fstu_aligned(wp_gate, 16) && fstu_aligned(wp_up, 16) && fstu_aligned(act, 8), FSTU_EALIGN,
               "fstu_glu_packed: pointers must be 16-byte aligned");
  GluArgs a = {};
  a.h = (const bf16_t*)h; a.wp_gate = (const uint4*)wp_gate; a.wp_up = (const uint4*)wp_up; a.act = (bf16_t*)act;
  a.rows = rows; a.d = d; a.I = I; a.ldh = ldh; a.ldact = ldact;
  return glu_launch(a, 0, 0, "fstu_glu_packed", (hipStream_t)stream);
}

extern "C" int fstu_glu_packed_norm(const void* x_in, const void* delta, void* x_out, const void* norm_w, float eps,
                                    const void* wp_gate, const void* wp_up, void* act, int ldact, int rows, int I, int d,
                                    void* stream) {
  FSTU_REQUIRE(x_in && norm_w && wp_gate && wp_up && act, FSTU_ENULL, "fstu_glu_packed_norm: null pointer");
  // 17..32 rows: the norm is formed in the matrix-core fragments (two row tiles) of a stream that already holds the
  // sub-layer's output (fstu_linear_packed_add, the recurrence step with a residual): no delta, nothing stored
  const bool wide = rows > FSTU_MAX_DECODE_ROWS;
  FSTU_REQUIRE(wide ? fstu_mlp_packed_rows32_supported(rows, d, I) : fstu_glu_packed_supported(rows, d, I), FSTU_ESHAPE,
               "fstu_glu_packed_norm: unsupported shape rows=%d d=%d I=%d", rows, d, I);
  FSTU_REQUIRE(!wide || (delta == nullptr && x_out == nullptr), FSTU_EARG,
               "fstu_glu_packed_norm: more than %d rows take the summed stream (delta and x_out must be NULL)", FSTU_MAX_DECODE_ROWS);
  FSTU_REQUIRE(ldact >= I && ldact % 4 == 0, FSTU_ESHAPE, "fstu_glu_packed_norm: ldact=%d", ldact);
  FSTU_REQUIRE(wide || x_out != x_in, FSTU_EARG, "fstu_glu_packed_norm: x_out must not alias x_in (other workgroups still read it)");
  FSTU_REQUIRE(fstu_aligned(x_in, 16) && fstu_aligned(delta, 16) && fstu_aligned(x_out, 16) && fstu_aligned(norm_w, 16) &&
                   fstu_aligned(wp_gate, 16) && fstu_aligned(wp_up, 16) && fstu_aligned(act, 8),
               FSTU_EALIGN, "fstu_glu_packed_norm: pointers must be 16-byte aligned");
  FSTU_REQUIRE(wide || (size_t)rows * (d + 8) * 2 <= 96 * 1024, FSTU_ESHAPE, "fstu_glu_packed_norm: rows*d too large for LDS");
  GluArgs a = {};
  a.wp_gate = (const uint4*)wp_gate; a.wp_up = (const uint4*)wp_up; a.act = (bf16_t*)act;
  a.rows = rows; a.d = d; a.I = I; a.ldh = d; a.ldact = ldact;
  a.x_in = (const bf16_t*)x_in; a.delta = delta; a.x_out = (bf16_t*)x_out; a.norm_w = (const bf16_t*)norm_w;
  a.eps = eps;
  return glu_launch(a, wide ? 3 : 1, 0, "fstu_glu_packed_norm", (hipStream_t)stream);
}

// y = T(x W^T) over packed W (N,K): x given normalised (norm_w == NULL, x = h with row stride ldx) or as the residual
// stream to normalise first (norm_w != NULL, rows dense): h = rmsnorm(x) * norm_w in the prologue.
extern "C" int fstu_linear_packed(const void* x, int ldx, const void* norm_w, float eps, const void* wp, void* y, int ldy,
                                  int rows, int N, int K, void* stream) {
  FSTU_REQUIRE(x && wp && y, FSTU_ENULL, "fstu_linear_packed: null pointer");
  // 17..32 rows: two row tiles; with norm_w the norm is formed in the matrix-core fragments
  const bool wide = rows > FSTU_MAX_DECODE_ROWS;
  FSTU_REQUIRE(fstu_glu_packed_supported(rows, K, N) ||
                   (rows <= 2 * FSTU_MAX_DECODE_ROWS && fstu_glu_packed_supported(FSTU_MAX_DECODE_ROWS, K, N)),
               FSTU_ESHAPE, "fstu_linear_packed: unsupported shape rows=%d K=%d N=%d", rows, K, N);
  FSTU_REQUIRE(ldx >= K && ldx % 8 == 0 && ldy >= N && ldy % 4 == 0, FSTU_ESHAPE, "fstu_linear_packed: ldx=%d ldy=%d", ldx, ldy);
  FSTU_REQUIRE(norm_w == nullptr || ldx == K, FSTU_ESHAPE, "fstu_linear_packed: the norm prologue needs dense rows");
  FSTU_REQUIRE(fstu_aligned(x, 16) && fstu_aligned(norm_w, 16) && fstu_aligned(wp, 16) && fstu_aligned(y, 8), FSTU_EALIGN,
               "fstu_linear_packed: pointers must be 16-byte aligned");
  FSTU_REQUIRE(norm_w == nullptr || wide || (size_t)rows * (K + 8) * 2 <= 96 * 1024, FSTU_ESHAPE, "fstu_linear_packed: rows*K too large for LDS");
  GluArgs a = {};
  a.wp_gate = (const uint4*)wp; a.wp_up = (const uint4*)wp; a.act = (bf16_t*)y;
  a.rows = rows; a.d = K; a.I = N; a.ldh = ldx; a.ldact = ldy; a.eps = eps;
  if (norm_w) { a.x_in = (const bf16_t*)x; a.norm_w = (const bf16_t*)norm_w; } else { a.h = (const bf16_t*)x; }
  return glu_launch(a, norm_w != nullptr ? (wide ? 3 : 1) : 0, 1, "fstu_linear_packed", (hipStream_t)stream);
}

// The same projection joining the residual stream: res_out = T(res_in + T(x W^T)), rows of stride N in both (res_out
// may be res_in: every pair is read and written by the same lane).  The launch that normalises the stream afterwards
// (fstu_glu_packed_norm at 17..32 rows) then needs no add of its own.
extern "C" int fstu_linear_packed_add(const void* x, int ldx, const void* wp, const void* res_in, void* res_out, int rows, int N,
                                      int K, void* stream) {
  FSTU_REQUIRE(x && wp && res_in && res_out, FSTU_ENULL, "fstu_linear_packed_add: null pointer");
  FSTU_REQUIRE(rows >= 1 && rows <= 2 * FSTU_MAX_DECODE_ROWS && fstu_glu_packed_supported(rows > FSTU_MAX_DECODE_ROWS ? FSTU_MAX_DECODE_ROWS : rows, K, N) &&
                   N % 8 == 0,
               FSTU_ESHAPE, "fstu_linear_packed_add: unsupported shape rows=%d K=%d N=%d", rows, K, N);
  FSTU_REQUIRE(ldx >= K && ldx % 8 == 0, FSTU_ESHAPE, "fstu_linear_packed_add: ldx=%d", ldx);
  FSTU_REQUIRE(fstu_aligned(x, 16) && fstu_aligned(wp, 16) && fstu_aligned(res_in, 4) && fstu_aligned(res_out, 4), FSTU_EALIGN,
               "fstu_linear_packed_add: x and wp must be 16-byte aligned, the residual rows 4");
  GluArgs a = {};
  a.wp_gate = (const uint4*)wp; a.wp_up = (const uint4*)wp; a.act = (bf16_t*)res_out; a.h = (const bf16_t*)x;
  a.rows = rows; a.d = K; a.I = N; a.ldh = ldx; a.ldact = N;
  a.x_in = (const bf16_t*)res_in; a.x_out = (bf16_t*)res_out;
  return glu_launch(a, 0, 1, "fstu_linear_packed_add", (hipStream_t)stream);
}

// The tied head over a packed embedding: logits = T(x W^T) for rows <= 32 and the rows' packed maxima at `temperature`
// into best_ws (rows x 64 words, zero on entry), as fstu_head_maxima leaves them.
extern "C" int fstu_head_maxima_packed(const void* x, int ldx, const void* wp, void* logits, int ldy, int rows, int N, int K,
                                       float temperature, void* best_ws, void* stream) {
  FSTU_REQUIRE(x && wp && logits && best_ws, FSTU_ENULL, "fstu_head_maxima_packed: null pointer");
  FSTU_REQUIRE(rows >= 1 && rows <= 2 * FSTU_MAX_DECODE_ROWS && fstu_glu_packed_supported(rows > FSTU_MAX_DECODE_ROWS ? FSTU_MAX_DECODE_ROWS : rows, K, N),
               FSTU_ESHAPE, "fstu_head_maxima_packed: unsupported shape rows=%d K=%d N=%d", rows, K, N);
  FSTU_REQUIRE(ldx >= K && ldx % 8 == 0 && ldy >= N && temperature > 0.f, FSTU_ESHAPE, "fstu_head_maxima_packed: ldx=%d ldy=%d temperature=%g",
               ldx, ldy, (double)temperature);
  FSTU_REQUIRE(fstu_aligned(x, 16) && fstu_aligned(wp, 16) && fstu_aligned(logits, 2) && fstu_aligned(best_ws, 8), FSTU_EALIGN,
               "fstu_head_maxima_packed: x and wp must be 16-byte aligned, best_ws 8");
  GluArgs a = {};
  a.wp_gate = (const uint4*)wp; a.wp_up = (const uint4*)wp; a.act = (bf16_t*)logits; a.h = (const bf16_t*)x;
  a.rows = rows; a.d = K; a.I = N; a.ldh = ldx; a.ldact = ldy;
  a.best = (unsigned long long*)best_ws; a.temperature = temperature;
  return glu_launch(a, 0, 2, "fstu_head_maxima_packed", (hipStream_t)stream);
}

// y = T(h W^T) with h = rmsnorm(x') * norm_w and x' = T(x_in + T(sum of nslices fp32 slices)): the add+norm launch
// between a split-K projection and the next projection, folded into the latter.  x' is stored to x_out by one
// workgroup (x_out must not alias x_in: the other workgroups still read it).
extern "C" int fstu_linear_packed_res(const void* x_in, const float* partial, int nslices, void* x_out, const void* norm_w,
                                      float eps, const void* wp, void* y, int ldy, int rows, int N, int K, void* stream) {
  FSTU_REQUIRE(x_in && partial && x_out && norm_w && wp && y, FSTU_ENULL, "fstu_linear_packed_res: null pointer");
  FSTU_REQUIRE((fstu_glu_packed_supported(rows, K, N) && NormPrologue<512, 2, 4>::supported(rows, K)), FSTU_ESHAPE,
               "fstu_linear_packed_res: unsupported shape rows=%d K=%d N=%d", rows, K, N);
  FSTU_REQUIRE(nslices >= 1 && nslices <= 4, FSTU_EARG, "fstu_linear_packed_res: nslices=%d outside 1..4", nslices);
  FSTU_REQUIRE(ldy >= N && ldy % 4 == 0, FSTU_ESHAPE, "fstu_linear_packed_res: ldy=%d", ldy);
  FSTU_REQUIRE(x_out != x_in, FSTU_EARG, "fstu_linear_packed_res: x_out must not alias x_in");
  FSTU_REQUIRE(fstu_aligned(x_in, 16) && fstu_aligned(partial, 16) && fstu_aligned(x_out, 16) && fstu_aligned(norm_w, 16) &&
                   fstu_aligned(wp, 16) && fstu_aligned(y, 8),
               FSTU_EALIGN, "fstu_linear_packed_res: pointers must be 16-byte aligned");
  FSTU_REQUIRE((size_t)rows * (K + 8) * 2 <= 96 * 1024, FSTU_ESHAPE, "fstu_linear_packed_res: rows*K too large for LDS");
  GluArgs a = {};
  a.wp_gate = (const uint4*)wp; a.wp_up = (const uint4*)wp; a.act = (bf16_t*)y;
  a.rows = rows; a.d = K; a.I = N; a.ldh = K; a.ldact = ldy; a.eps = eps;
  a.x_in = (const bf16_t*)x_in; a.delta = partial; a.nslices = nslices; a.x_out = (bf16_t*)x_out; a.norm_w = (const bf16_t*)norm_w;
  return glu_launch(a, 2, 1, "fstu_linear_packed_res", (hipStream_t)stream);
}

// Balanced split-K down projection: partial (ksplit, rows, d) fp32 slices, summed by fstu_add_rmsnorm(delta_mode 1).
// Returns the number of slices through *ksplit_out (16, the K chunks of the launch).
extern "C" int fstu_down_packed_splitk(const void* act, int ldact, const void* wp_down, float* partial, int rows, int d, int I,
                                       int* ksplit_io, void* stream) {
  FSTU_REQUIRE(act && wp_down && partial, FSTU_ENULL, "fstu_down_packed_splitk: null pointer");
  // *ksplit_io on entry: the number of K slices wanted (4, 8 or 16; anything else: 16); on return: the number written
  const int want = ksplit_io ? *ksplit_io : 16;
  const int KS = (want == 4 || want == 8) ? want : 16;
  FSTU_REQUIRE(rows >= 1 && rows <= 2 * FSTU_MAX_DECODE_ROWS && d >= 16 && d % 16 == 0 && I >= KS * 32 && I % (KS * 32) == 0 &&
                   (size_t)I * d * 2 < 0xfff00000ull && (size_t)rows * ldact * 2 < 0x7ff00000ull,
               FSTU_ESHAPE, "fstu_down_packed_splitk: unsupported shape rows=%d d=%d I=%d", rows, d, I);
  FSTU_REQUIRE(ldact >= I && ldact % 8 == 0, FSTU_ESHAPE, "fstu_down_packed_splitk: ldact=%d", ldact);
  FSTU_REQUIRE(fstu_aligned(act, 16) && fstu_aligned(wp_down, 16) && fstu_aligned(partial, 16), FSTU_EALIGN,
               "fstu_down_packed_splitk: pointers must be 16-byte aligned");
  int cus = query_cus();
  FSTU_REQUIRE(cus > 0, FSTU_EARG, "fstu_down_packed_splitk: no device");
  DownSkArgs a;
  a.act = (const bf16_t*)act; a.wp_down = (const uint4*)wp_down; a.partial = partial;
  a.rows = rows; a.d = d; a.I = I; a.ldact = ldact; a.KS = KS; a.tiles_out = d / 16; a.kch = I / 32 / KS;
  int ngroups = cus / KS;
  if (ngroups < 1) ngroups = 1;
  if (ngroups > a.tiles_out) ngroups = a.tiles_out;
  a.tpw = (a.tiles_out + ngroups - 1) / ngroups;
  ngroups = (a.tiles_out + a.tpw - 1) / a.tpw;
  const int ksb = (a.kch + 7) / 8;
  FSTU_REQUIRE(ksb <= 12, FSTU_ESHAPE, "fstu_down_packed_splitk: I=%d too large", I);
  dim3 grid(ngroups * KS);
  hipStream_t s = (hipStream_t)stream;
#define DOWN_GO(KSB)                                                                                                          \
  do {                                                                                                                         \
    if (rows > FSTU_MAX_DECODE_ROWS)                                                                                           \
      hipLaunchKernelGGL((down_splitk_balanced_kernel<KSB, 2>), grid, dim3(512), 0, s, a.act, a.wp_down, a.partial, a.rows, a.d, \
                         a.I, a.ldact, a.KS, a.tpw, a.tiles_out, a.kch);                                                       \
    else                                                                                                                       \
      hipLaunchKernelGGL((down_splitk_balanced_kernel<KSB, 1>), grid, dim3(512), 0, s, a.act, a.wp_down, a.partial, a.rows, a.d, \
                         a.I, a.ldact, a.KS, a.tpw, a.tiles_out, a.kch);                                                       \
  } while (0)
  if (ksb <= 1) DOWN_GO(1);
  else if (ksb == 2) DOWN_GO(2);
  else if (ksb == 3) DOWN_GO(3);
  else if (ksb == 4) DOWN_GO(4);
  else if (ksb <= 6) DOWN_GO(6);
  else if (ksb <= 8) DOWN_GO(8);
  else if (ksb == 9) DOWN_GO(9);
  else DOWN_GO(12);
#undef DOWN_GO
  FSTU_CHECK_LAUNCH("fstu_down_packed_splitk");
  if (ksplit_io) *ksplit_io = KS;
  return FSTU_OK;
}
