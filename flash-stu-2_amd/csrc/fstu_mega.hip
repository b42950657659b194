// One decode step of the whole layer stack as ONE persistent launch (bf16, recurrence STU state).
//
// A kernel boundary costs a dependent decode step about 3 us of launch plus a cold first trip to memory, 51 times per
// token.  Here one grid of G workgroups (one per CU, all resident) walks the step as a sequence of phases, and what one
// phase hands to the next moves through device memory as TAGGED 64-bit words: the low half carries the payload (two
// bf16 values or one fp32), the high half the tag of the producing phase, (epoch << 8) | phase.  A consumer polls the
// words it needs with relaxed agent-scope loads (coherent across the XCDs without cache flushes) until every tag
// matches: data and "ready" flag arrive in the same trip, there are no counters, no atomics on shared addresses and no
// grid barrier.  Weight loads of a phase are issued before its inputs are polled, so they stream while the workgroup
// waits.  Every spin is bounded: on a timeout the workgroup raises the abort word, every workgroup sees it at its next
// poll and the kernel exits normally (the host reads the error word).
//
// Phases per STU layer (flash_stu/layers/stu_layer.py:78-97 for one token):
//   S1  d/16 workgroups: h = rmsnorm(x) * w1, x_proj tile = h M_inputs (MFMA), recurrence step of the tile's 16 channels
//       (both parity banks, plus and minus branch rounded separately), x' = T(x + y)                -> X
//   S2  all: h = rmsnorm(x') * w_mlp, gate/up features of the workgroup, act = T(gelu(g)) * u        -> ACT
//   S3  all: (tile group, K chunk) of the down projection, fp32 partial tiles                        -> PART
//   S4  d/16 workgroups: x'' = T(x' + T(sum of the K chunks in order))                               -> X
// per attention layer (flash_stu/layers/attention_layer.py:50-66, flash_stu/modules/attention.py:59-105):
//   A1  3d/16 tiles: h = rmsnorm(x) * w1, qkv tile                                                   -> QKV
//   A2  B*H workgroups: ring append, one query against the window's keys, softmax, P.V               -> ATT
//   A3  d/16 workgroups: x' = T(x + T(att W_proj^T))                                                 -> X
//   then S2, S3, S4.
// Final: F1 all: h = rmsnorm(x) * w_f, logits of the workgroup's vocabulary tiles (+ packed row maxima -> BEST);
//        F2 workgroup 0: greedy token per row, position / step / epoch advanced.
#include <type_traits>
#include <mutex>
#include <vector>
#include "fstu_common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

#define MG_THREADS 512
#define MG_OOB 0xfffffff0u
#define MG_SPIN_LIMIT (1 << 15)     // polls of one wait (a poll is a trip to memory, about a microsecond)
#define MG_NB 4                     // reduction slots (tiles in flight per batch)
#define MG_KD 6                     // k steps per wave and tile of the down projection, at most
#define MG_NBD 3                    // down-projection tiles in flight per batch
#define MG_CTRL_EPOCH 0
#define MG_CTRL_ERR 32
#define MG_CTRL_ABORT 64

struct MegaLayer {
  int kind, pad;
  const bf16_t* norm1_w;
  const bf16_t* mlp_norm_w;
  const uint4* wp_first;    // packed M_inputs^T (d,d) or packed c_attn (3d,d)
  const uint4* wp_proj;     // packed c_proj (d,d)
  const uint4* wp_gate;
  const uint4* wp_up;
  const uint4* wp_down;
  float* state;
  const float* a;
  const float* ce;
  const float* co;
  bf16_t* kring;
  bf16_t* vring;
  const float* slopes;
};

struct MegaArgs {
  const MegaLayer* layers;
  const bf16_t* emb;
  const uint4* wp_emb;
  const bf16_t* final_norm_w;
  u64* xbuf[2];
  u64* qkv;
  u64* att;
  u64* act;
  u64* part;
  u64* best;
  unsigned* ctrl;
  bf16_t* logits;
  int64_t* tokens;     // column 0 of the token buffer (read at column pos)
  int64_t* tok_out;    // column 0 of the output view (written at column pos)
  int* dyn;            // device {position, sampling step} or NULL
  long long tok_stride;
  int n_layers, B, d, I, V, H, hd, window, cap, S, pos, greedy, ks_down;
  float eps, softcap, temperature;
};

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ __forceinline__ u64 ld_agent(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(u64* p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned ld_agent32(const unsigned* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent32(unsigned* p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, p ? (unsigned)bytes : 0u, 0x00020000);
}
// weights are read exactly once: non-temporal, so the stream does not push the exchange buffers out of the L2
__device__ __forceinline__ uint4 buf_load16_stream(rsrc_t rs, unsigned off) {
  u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 2);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float lo_bf16(unsigned w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi_bf16(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float rnd_bf16(float v) { return bf16_to_f32(f32_to_bf16(v)); }

__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  const float e = __builtin_amdgcn_exp2f(2.8853900817779268f * inner);   // exp(2 inner)
  const float th = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
  return 0.5f * x * (1.0f + th);
}

// monotone 32-bit key of a float (larger float <=> larger key)
__device__ __forceinline__ unsigned f32_okey(float v) {
  const unsigned u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

template <int KPW, int NXW>
__global__ void __launch_bounds__(MG_THREADS)
mega_step_kernel(const MegaArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  // The thread's coordinates are re-derived from an opaque copy of the thread index at the start of every phase
  // (MG_PHASE): otherwise the compiler hoists every per-thread address computation of all phases out of the layer loop
  // and keeps hundreds of registers alive across it (spills on the critical path of every phase).
  int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  int r = lane & 15, g = lane >> 4;
#define MG_PHASE()                          \
  do {                                      \
    asm volatile("" : "+v"(tid));           \
    lane = tid & 63; w = tid >> 6;          \
    r = lane & 15; g = lane >> 4;           \
    xrow = r < B;                           \
  } while (0)
  const int wg = blockIdx.x, G = gridDim.x;
  const int B = a.B, d = a.d, I = a.I;
  const int ld = d + 8;
  const int hw = d >> 1;                       // tagged words per row of x
  const int nxw = B * hw;                      // words of x
  const int cpr = d >> 7;                      // 64-word chunks per row
  // ---- LDS
  bf16_t* hs = (bf16_t*)smem;                                          // B x ld normalised rows
  float* red = (float*)(smem + (((size_t)B * ld * 2 + 15) & ~(size_t)15));   // MG_NB x 8 x 256 floats
  float* ssp = red + MG_NB * 8 * 256;                                  // B * cpr partial sums of squares (<= 256)
  float* xt = ssp + 256;                                               // 16 x 16 own tile of the residual stream
  float* xps = xt + 256;                                               // 16 x 16 projected inputs of the tile
  float* misc = xps + 256;                                             // 64 floats
  bool xrow = r < B;
  const int pos = a.dyn ? a.dyn[0] : a.pos;
  const unsigned epoch = a.ctrl[MG_CTRL_EPOCH];
  const unsigned tbase = epoch << 8;
  unsigned ph = 0;
  const int ksteps = d >> 5;
  const int mytile = wg;                        // tile of the residual stream this workgroup updates (wg < d/16)

  // leaves the kernel (all threads) when `bad` holds anywhere in the workgroup
#define MG_CHECK(bad)                                                        \
  do {                                                                       \
    if (__syncthreads_or((bad) ? 1 : 0)) {                                   \
      if (tid == 0) {                                                        \
        st_agent32(a.ctrl + MG_CTRL_ABORT, 1u);                              \
        st_agent32(a.ctrl + MG_CTRL_ERR, 0x100u + ph);                       \
      }                                                                      \
      return;                                                                \
    }                                                                        \
  } while (0)

  // ---------------------------------------------------------------- residual rows in registers
  unsigned xw[NXW];     // word tid + 512*i of x: two bf16
  // polls `n` tagged words (word tid + 512*i for i < CNT) until every tag matches; payloads to out[]
  auto poll = [&](const u64* buf, int n, unsigned tag, unsigned* out, auto cnt_tag) -> bool {
    constexpr int CNT = decltype(cnt_tag)::value;
    u64 v[CNT];
    int spins = 0;
    bool bad = false;
    // A workgroup that arrives early probes ONE word per thread, with a pause between the probes: while a phase of few
    // workgroups runs, the others wait here, and polling everything at full rate floods the memory system that the
    // running phase depends on.  Once the probe word is there, the rest is there as well or about to be.
    for (;;) {
      v[0] = tid < n ? ld_agent(buf + tid) : ((u64)tag << 32);
      if ((unsigned)(v[0] >> 32) == tag) break;
      if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
      __builtin_amdgcn_s_sleep(2);
    }
    if (CNT > 1 && !bad) {
      for (;;) {
        bool ok = true;
#pragma unroll
        for (int i = 1; i < CNT; ++i) {
          const int idx = tid + MG_THREADS * i;
          v[i] = idx < n ? ld_agent(buf + idx) : ((u64)tag << 32);
        }
#pragma unroll
        for (int i = 1; i < CNT; ++i) ok = ok && (unsigned)(v[i] >> 32) == tag;
        if (ok) break;
        if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
      }
    }
#pragma unroll
    for (int i = 0; i < CNT; ++i) out[i] = (unsigned)v[i];
    return bad;
  };

  // h = T((x * rstd) * w) of every row into hs; the workgroup's own tile of x into xt
  auto norm_rows = [&](const bf16_t* __restrict__ nw) {
    unsigned nwv[NXW];
#pragma unroll
    for (int i = 0; i < NXW; ++i) {
      const int idx = tid + MG_THREADS * i;
      const int chunk = idx >> 6, row = chunk / cpr;
      const int c2 = idx - row * hw;
      nwv[i] = idx < nxw ? *(const unsigned*)(nw + 2 * c2) : 0u;
      float ss = 0.f;
      if (idx < nxw) { const float lo = lo_bf16(xw[i]), hi = hi_bf16(xw[i]); ss = fmaf(lo, lo, hi * hi); }
      ss = wave_sum(ss);
      if (lane == 0 && chunk < B * cpr) ssp[chunk] = ss;
    }
    __syncthreads();
    const float inv_d = 1.0f / (float)d;
#pragma unroll
    for (int i = 0; i < NXW; ++i) {
      const int idx = tid + MG_THREADS * i;
      if (idx < nxw) {
        const int chunk = idx >> 6, row = chunk / cpr;
        const int c2 = idx - row * hw;
        float ss = 0.f;
        for (int k = 0; k < cpr; ++k) ss += ssp[row * cpr + k];
        const float rstd = rsqrtf(ss * inv_d + a.eps);
        const float lo = lo_bf16(xw[i]), hi = hi_bf16(xw[i]);
        *(unsigned*)(hs + (size_t)row * ld + 2 * c2) = pack2_bf16((lo * rstd) * lo_bf16(nwv[i]), (hi * rstd) * hi_bf16(nwv[i]));
        if (((2 * c2) >> 4) == mytile) { xt[row * 16 + ((2 * c2) & 15)] = lo; xt[row * 16 + ((2 * c2) & 15) + 1] = hi; }
      }
    }
    __syncthreads();
  };

  // this wave's activation fragments (B operand) for its KPW k steps
  auto load_xb = [&](uint4 (&xb)[KPW]) {
#pragma unroll
    for (int u = 0; u < KPW; ++u)
      xb[u] = xrow ? *(const uint4*)(hs + (size_t)r * ld + (w * KPW + u) * 32 + g * 8) : make_uint4(0, 0, 0, 0);
  };

  // D layout of a 16x16 tile: lane (r, g) holds features 4g+i of batch row r.  The 8 K shares of slot `slot` in wave order.
  auto reduce_slot = [&](int slot, float (&o)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const float4 p = *(const float4*)(red + ((size_t)(slot * 8 + s) * 64 + lane) * 4);
      o[0] += p.x; o[1] += p.y; o[2] += p.z; o[3] += p.w;
    }
  };
  auto stash = [&](int slot, floatx4_t acc) {
    *(float4*)(red + ((size_t)(slot * 8 + w) * 64 + lane) * 4) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  };

  // ---------------------------------------------------------------- embedding rows of the input tokens
  {
#pragma unroll
    for (int i = 0; i < NXW; ++i) {
      const int idx = tid + MG_THREADS * i;
      xw[i] = 0u;
      if (idx < nxw) {
        const int row = (idx >> 6) / cpr, c2 = idx - row * hw;
        long long t = a.tokens[(size_t)row * a.tok_stride + pos];
        t = t < 0 ? 0 : (t >= a.V ? a.V - 1 : t);
        xw[i] = *(const unsigned*)(a.emb + (size_t)t * d + 2 * c2);
      }
    }
  }
  bool have_x = true;       // xw holds the current residual rows (no poll needed)
  int xsel = 0;             // exchange buffer of the latest residual rows
  unsigned tag_x = 0;

  const int tiles_d = d >> 4;
  // features of the gate/up projection owned by this workgroup, in half tiles of 8
  const int nhalf = I >> 3;
  const int h0 = (int)(((long long)wg * nhalf) / G), h1 = (int)(((long long)(wg + 1) * nhalf) / G);
  // down projection: (tile group, K chunk)
  const int KS = a.ks_down, ntg = G / KS;
  const int dchunk = wg % KS, dgrp = wg / KS;
  const int tpg = (tiles_d + ntg - 1) / ntg;
  const int kst_I = I >> 5, kch = kst_I / KS;

  for (int l = 0; l < a.n_layers; ++l) {
    const MegaLayer& L = a.layers[l];
    const int parity = pos & 1;
    if (L.kind == 0) {
      // ============================================================ S1: projection + recurrence step, tile `wg`
      MG_PHASE();
      const unsigned tag_out = tbase | (++ph);
      if (wg < tiles_d) {
        const int c0 = wg * 16;
        // recurrence operands: they depend on nothing, so they go out first
        const int sb = tid >> 6, cq = tid & 3, jsub = (tid >> 2) & 15;
        const int S = a.S;
        float4 he[2][4], ho[2][4], cev[4], cov[4];
        float av[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int j = min(jsub + 16 * k, S - 1);
          cev[k] = *(const float4*)(L.ce + (size_t)j * d + c0 + 4 * cq);
          cov[k] = *(const float4*)(L.co + (size_t)j * d + c0 + 4 * cq);
          av[k] = L.a[j];
#pragma unroll
          for (int bb = 0; bb < 2; ++bb) {
            const int b = min(sb + 8 * bb, B - 1);
            he[bb][k] = *(const float4*)(L.state + (((size_t)b * 2 + parity) * S + j) * d + c0 + 4 * cq);
            ho[bb][k] = *(const float4*)(L.state + (((size_t)b * 2 + (parity ^ 1)) * S + j) * d + c0 + 4 * cq);
          }
        }
        // projection weights of the tile
        const rsrc_t rw = make_rsrc(L.wp_first, (size_t)tiles_d * ksteps * 1024);
        uint4 wa[KPW];
#pragma unroll
        for (int u = 0; u < KPW; ++u) wa[u] = buf_load16_stream(rw, (unsigned)(((wg * ksteps + w * KPW + u) * 64 + lane) * 16));
        if (!have_x) {
          const bool bad = poll(a.xbuf[xsel], nxw, tag_x, xw, std::integral_constant<int, NXW>());
          MG_CHECK(bad);
        }
        norm_rows(L.norm1_w);
        uint4 xb[KPW];
        load_xb(xb);
        floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KPW; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
        stash(0, acc);
        __syncthreads();
        if (w == 0) {
          float o[4];
          reduce_slot(0, o);
#pragma unroll
          for (int i = 0; i < 4; ++i) xps[r * 16 + 4 * g + i] = rnd_bf16(o[i]);
        }
        __syncthreads();
        // recurrence step: thread (batch row sb [+8], channel quad cq, mode group jsub)
#pragma unroll
        for (int bb = 0; bb < 2; ++bb) {
          const int b = sb + 8 * bb;
          if (b < B) {     // uniform per wave
            const float x0 = xps[b * 16 + 4 * cq], x1 = xps[b * 16 + 4 * cq + 1], x2 = xps[b * 16 + 4 * cq + 2], x3 = xps[b * 16 + 4 * cq + 3];
            float4 E = make_float4(0.f, 0.f, 0.f, 0.f), Od = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int j = jsub + 16 * k;
              if (j < S) {
                float4 hv = he[bb][k];
                hv.x = fmaf(av[k], hv.x, x0);
                hv.y = fmaf(av[k], hv.y, x1);
                hv.z = fmaf(av[k], hv.z, x2);
                hv.w = fmaf(av[k], hv.w, x3);
                *(float4*)(L.state + (((size_t)b * 2 + parity) * S + j) * d + c0 + 4 * cq) = hv;
                E.x = fmaf(cev[k].x, hv.x, E.x); E.y = fmaf(cev[k].y, hv.y, E.y);
                E.z = fmaf(cev[k].z, hv.z, E.z); E.w = fmaf(cev[k].w, hv.w, E.w);
                const float4 hq = ho[bb][k];
                Od.x = fmaf(cov[k].x, hq.x, Od.x); Od.y = fmaf(cov[k].y, hq.y, Od.y);
                Od.z = fmaf(cov[k].z, hq.z, Od.z); Od.w = fmaf(cov[k].w, hq.w, Od.w);
              }
            }
            // modes beyond 64 (S > 64): the remaining groups straight from memory
            for (int j = jsub + 64; j < S; j += 16) {
              float* sp = L.state + (((size_t)b * 2 + parity) * S + j) * d + c0 + 4 * cq;
              float4 hv = *(float4*)sp;
              const float aj = L.a[j];
              const float4 cj = *(const float4*)(L.ce + (size_t)j * d + c0 + 4 * cq);
              hv.x = fmaf(aj, hv.x, x0); hv.y = fmaf(aj, hv.y, x1); hv.z = fmaf(aj, hv.z, x2); hv.w = fmaf(aj, hv.w, x3);
              *(float4*)sp = hv;
              E.x = fmaf(cj.x, hv.x, E.x); E.y = fmaf(cj.y, hv.y, E.y); E.z = fmaf(cj.z, hv.z, E.z); E.w = fmaf(cj.w, hv.w, E.w);
              const float4 hq = *(const float4*)(L.state + (((size_t)b * 2 + (parity ^ 1)) * S + j) * d + c0 + 4 * cq);
              const float4 oj = *(const float4*)(L.co + (size_t)j * d + c0 + 4 * cq);
              Od.x = fmaf(oj.x, hq.x, Od.x); Od.y = fmaf(oj.y, hq.y, Od.y); Od.z = fmaf(oj.z, hq.z, Od.z); Od.w = fmaf(oj.w, hq.w, Od.w);
            }
            // sum over the 16 mode groups: lane bits 2..5
#pragma unroll
            for (int o = 4; o < 64; o <<= 1) {
              E.x += __shfl_xor(E.x, o, 64); E.y += __shfl_xor(E.y, o, 64); E.z += __shfl_xor(E.z, o, 64); E.w += __shfl_xor(E.w, o, 64);
              Od.x += __shfl_xor(Od.x, o, 64); Od.y += __shfl_xor(Od.y, o, 64); Od.z += __shfl_xor(Od.z, o, 64); Od.w += __shfl_xor(Od.w, o, 64);
            }
            if (jsub == 0) {
              const float y0 = rnd_bf16(rnd_bf16(E.x + Od.x) + rnd_bf16(E.x - Od.x)), y1 = rnd_bf16(rnd_bf16(E.y + Od.y) + rnd_bf16(E.y - Od.y));
              const float y2 = rnd_bf16(rnd_bf16(E.z + Od.z) + rnd_bf16(E.z - Od.z)), y3 = rnd_bf16(rnd_bf16(E.w + Od.w) + rnd_bf16(E.w - Od.w));
              const float* xr = xt + b * 16 + 4 * cq;
              u64* dst = a.xbuf[xsel ^ 1] + (((size_t)b * d + c0 + 4 * cq) >> 1);
              st_agent(dst, ((u64)tag_out << 32) | pack2_bf16(xr[0] + y0, xr[1] + y1));
              st_agent(dst + 1, ((u64)tag_out << 32) | pack2_bf16(xr[2] + y2, xr[3] + y3));
            }
          }
        }
      }
      xsel ^= 1;
      tag_x = tag_out;
      have_x = false;
    } else {
      // ============================================================ A1: QKV projection tiles
      MG_PHASE();
      const unsigned tag_qkv = tbase | (++ph);
      const int tiles_q = 3 * tiles_d;
      const int nact = min(tiles_q, G);
      const int qt0 = (int)(((long long)wg * tiles_q) / nact), qt1 = wg < nact ? (int)(((long long)(wg + 1) * tiles_q) / nact) : qt0;
      if (wg < nact) {
        const rsrc_t rw = make_rsrc(L.wp_first, (size_t)tiles_q * ksteps * 1024);
        uint4 wa[2][KPW];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int u = 0; u < KPW; ++u)
            wa[j][u] = buf_load16_stream(rw, qt0 + j < qt1 ? (unsigned)((((qt0 + j) * ksteps + w * KPW + u) * 64 + lane) * 16) : MG_OOB);
        if (!have_x) {
          const bool bad = poll(a.xbuf[xsel], nxw, tag_x, xw, std::integral_constant<int, NXW>());
          MG_CHECK(bad);
          have_x = true;
        }
        norm_rows(L.norm1_w);
        uint4 xb[KPW];
        load_xb(xb);
        for (int t0 = qt0; t0 < qt1; t0 += 2) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < KPW; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[j][u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
            stash(j, acc);
#pragma unroll
            for (int u = 0; u < KPW; ++u)
              wa[j][u] = buf_load16_stream(rw, t0 + 2 + j < qt1 ? (unsigned)((((t0 + 2 + j) * ksteps + w * KPW + u) * 64 + lane) * 16) : MG_OOB);
          }
          __syncthreads();
          if (w < 2 && t0 + w < qt1) {
            float o[4];
            reduce_slot(w, o);
            if (xrow) {
              u64* dst = a.qkv + (((size_t)r * 3 * d + (t0 + w) * 16 + 4 * g) >> 1);
              st_agent(dst, ((u64)tag_qkv << 32) | pack2_bf16(o[0], o[1]));
              st_agent(dst + 1, ((u64)tag_qkv << 32) | pack2_bf16(o[2], o[3]));
            }
          }
          __syncthreads();
        }
      }
      // ============================================================ A2: attention of (batch row, head) = wg
      MG_PHASE();
      const unsigned tag_att = tbase | (++ph);
      const int H = a.H, hd = a.hd;
      // the output projection's weights go out before the attention phase: they depend on nothing
      uint4 wpj[KPW];
      {
        const rsrc_t rp = make_rsrc(L.wp_proj, (size_t)tiles_d * ksteps * 1024);
#pragma unroll
        for (int u = 0; u < KPW; ++u) wpj[u] = buf_load16_stream(rp, wg < tiles_d ? (unsigned)(((wg * ksteps + w * KPW + u) * 64 + lane) * 16) : MG_OOB);
      }
      for (int unit = wg; unit < B * H; unit += G) {
        const int b = unit / H, h = unit - b * H;
        const int LPK = hd >> 3;                       // lanes per key (16 bytes each)
        const int KP = MG_THREADS / LPK;               // keys per pass
        const int kl = tid / LPK, dl = tid - kl * LPK;
        const int lo = max(0, pos - a.window);
        const int nring = pos - lo;                    // keys read from the ring: positions lo .. pos-1
        const size_t hbase = ((size_t)b * H + h) * a.cap * hd;
        float* qs = misc;                              // q, k, v of the new token: 3 * hd floats (hd <= 128: 384)
        float* sc = red;                               // scores (<= cap + 1 floats)
        float* part = red + 2048;                      // KP x hd partial outputs
        // ring loads first (they do not depend on this step's q)
        constexpr int NP = 9;                          // passes held in registers at once
        const int slot_lo = lo % a.cap;
        auto slot_of = [&](int j) { int s = slot_lo + (j - lo); return s >= a.cap ? s - a.cap : s; };
        uint4 kv[NP], vv[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
          const int j = lo + kl + p * KP;
          const int s = slot_of(min(j, max(pos - 1, lo)));
          kv[p] = *(const uint4*)(L.kring + hbase + (size_t)s * hd + dl * 8);
          vv[p] = *(const uint4*)(L.vring + hbase + (size_t)s * hd + dl * 8);
        }
        // q, k, v of this (row, head): 3 * hd / 2 tagged words
        {
          const int nwq = (3 * hd) >> 1;
          unsigned out1[1];
          u64 v = 0;
          int spins = 0;
          bool bad = false;
          const int part3 = tid / (hd >> 1), wi = tid - part3 * (hd >> 1);     // 0: q, 1: k, 2: v
          const u64* src = a.qkv + (((size_t)b * 3 * d + (size_t)part3 * d + h * hd) >> 1) + wi;
          if (tid < nwq) {
            for (;;) {
              v = ld_agent(src);
              if ((unsigned)(v >> 32) == tag_qkv) break;
              if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
              __builtin_amdgcn_s_sleep(2);
            }
            out1[0] = (unsigned)v;
            qs[part3 * hd + 2 * wi] = lo_bf16(out1[0]);
            qs[part3 * hd + 2 * wi + 1] = hi_bf16(out1[0]);
          }
          MG_CHECK(bad);
        }
        // ring append of the new token's key and value (slot pos % cap is not among the slots read above)
        if (tid < 2 * LPK) {
          const int which = tid / LPK, dd = tid - which * LPK;
          const float* srcf = qs + (1 + which) * hd + dd * 8;
          uint4 pk = make_uint4(pack2_bf16(srcf[0], srcf[1]), pack2_bf16(srcf[2], srcf[3]), pack2_bf16(srcf[4], srcf[5]), pack2_bf16(srcf[6], srcf[7]));
          bf16_t* ring = which ? L.vring : L.kring;
          *(uint4*)(ring + hbase + (size_t)(pos % a.cap) * hd + dd * 8) = pk;
        }
        float q8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q8[i] = qs[dl * 8 + i];
        const float scale = rsqrtf((float)hd), slope = L.slopes[h];
        const float inv_cap2l = a.softcap > 0.f ? 2.8853900817779268f / a.softcap : 0.f;
        auto score_of = [&](float dot, int j) {
          float s = dot * scale;
          if (a.softcap > 0.f) {
            const float e = __builtin_amdgcn_exp2f(s * inv_cap2l);
            s = a.softcap - (2.0f * a.softcap) * __builtin_amdgcn_rcpf(e + 1.0f);
          }
          return s - slope * (float)(pos - j);
        };
        auto dot8 = [&](uint4 kk) {
          const unsigned kw[4] = {kk.x, kk.y, kk.z, kk.w};
          float s = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) { s = fmaf(q8[2 * i], lo_bf16(kw[i]), s); s = fmaf(q8[2 * i + 1], hi_bf16(kw[i]), s); }
          for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, 64);
          return s;
        };
        // scores of the ring keys (passes beyond the registers re-load) and of the token itself
        for (int p0 = 0; p0 * KP < nring; p0 += NP) {
#pragma unroll
          for (int p = 0; p < NP; ++p) {
            const int j = lo + kl + (p0 + p) * KP;
            uint4 kk = kv[p];
            if (p0 > 0) kk = *(const uint4*)(L.kring + hbase + (size_t)slot_of(min(j, max(pos - 1, lo))) * hd + dl * 8);
            const float s = dot8(kk);
            if (j < pos && dl == 0) sc[j - lo] = score_of(s, j);
          }
        }
        if (kl == 0) {
          float s = 0.f;
#pragma unroll
          for (int i = 0; i < 8; ++i) s = fmaf(q8[i], qs[hd + dl * 8 + i], s);
          for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, 64);
          if (dl == 0) sc[nring] = score_of(s, pos);
        }
        __syncthreads();
        const int nk = nring + 1;
        float m = -INFINITY;
        for (int i = tid; i < nk; i += MG_THREADS) m = fmaxf(m, sc[i]);
        m = wave_max(m);
        if (lane == 0) misc[384 + w] = m;
        __syncthreads();
        m = misc[384];
#pragma unroll
        for (int i = 1; i < 8; ++i) m = fmaxf(m, misc[384 + i]);
        float lsum = 0.f;
        for (int i = tid; i < nk; i += MG_THREADS) { const float p = __expf(sc[i] - m); sc[i] = p; lsum += p; }
        lsum = wave_sum(lsum);
        __syncthreads();
        if (lane == 0) misc[392 + w] = lsum;
        __syncthreads();
        lsum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) lsum += misc[392 + i];
        // P.V: thread (key lane kl, 8 dims dl)
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        for (int p0 = 0; p0 * KP < nring; p0 += NP) {
#pragma unroll
          for (int p = 0; p < NP; ++p) {
            const int j = lo + kl + (p0 + p) * KP;
            uint4 v4 = vv[p];
            if (p0 > 0) v4 = *(const uint4*)(L.vring + hbase + (size_t)slot_of(min(j, max(pos - 1, lo))) * hd + dl * 8);
            const float pj = j < pos ? sc[j - lo] : 0.f;
            const unsigned vw[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) { acc[2 * i] = fmaf(pj, lo_bf16(vw[i]), acc[2 * i]); acc[2 * i + 1] = fmaf(pj, hi_bf16(vw[i]), acc[2 * i + 1]); }
          }
        }
        if (kl == 0) {
          const float ps = sc[nring];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[i] = fmaf(ps, qs[2 * hd + dl * 8 + i], acc[i]);
        }
        __syncthreads();      // scores are no longer needed by anyone below; part does not overlap them
#pragma unroll
        for (int i = 0; i < 8; ++i) part[kl * hd + dl * 8 + i] = acc[i];
        __syncthreads();
        if (tid < (hd >> 1)) {
          float s0 = 0.f, s1 = 0.f;
          for (int k = 0; k < KP; ++k) { s0 += part[k * hd + 2 * tid]; s1 += part[k * hd + 2 * tid + 1]; }
          const float inv = 1.0f / lsum;
          st_agent(a.att + (((size_t)b * d + h * hd) >> 1) + tid, ((u64)tag_att << 32) | pack2_bf16(s0 * inv, s1 * inv));
        }
        __syncthreads();
      }
      // ============================================================ A3: output projection + residual, tile `wg`
      MG_PHASE();
      const unsigned tag_out = tbase | (++ph);
      if (wg < tiles_d) {
        unsigned aw[NXW];
        const bool bad = poll(a.att, nxw, tag_att, aw, std::integral_constant<int, NXW>());
        MG_CHECK(bad);
        // attention rows into hs as they are (no norm)
#pragma unroll
        for (int i = 0; i < NXW; ++i) {
          const int idx = tid + MG_THREADS * i;
          if (idx < nxw) {
            const int row = (idx >> 6) / cpr, c2 = idx - row * hw;
            *(unsigned*)(hs + (size_t)row * ld + 2 * c2) = aw[i];
          }
        }
        __syncthreads();
        uint4 xb[KPW];
        load_xb(xb);
        floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KPW; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wpj[u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
        stash(0, acc);
        __syncthreads();
        if (w == 0) {
          float o[4];
          reduce_slot(0, o);
          if (xrow) {
            const float* xr = xt + r * 16 + 4 * g;
            u64* dst = a.xbuf[xsel ^ 1] + (((size_t)r * d + wg * 16 + 4 * g) >> 1);
            st_agent(dst, ((u64)tag_out << 32) | pack2_bf16(xr[0] + rnd_bf16(o[0]), xr[1] + rnd_bf16(o[1])));
            st_agent(dst + 1, ((u64)tag_out << 32) | pack2_bf16(xr[2] + rnd_bf16(o[2]), xr[3] + rnd_bf16(o[3])));
          }
        }
        __syncthreads();
      }
      xsel ^= 1;
      tag_x = tag_out;
      have_x = false;
    }

    // ============================================================== S2: gate/up projection + GLU, half tiles [h0, h1)
    MG_PHASE();
    const unsigned tag_act = tbase | (++ph);
    {
      const int gt0 = h0 >> 1, gt1 = (h1 + 1) >> 1;
      const int tiles_I = I >> 4;
      const rsrc_t rg = make_rsrc(L.wp_gate, (size_t)tiles_I * ksteps * 1024), ru = make_rsrc(L.wp_up, (size_t)tiles_I * ksteps * 1024);
      uint4 wa[2][KPW], wb[2][KPW];
      auto load_glu = [&](int j, int tile) {
        const int half = 2 * tile + (r >> 3);
        const bool ok = tile < gt1 && half >= h0 && half < h1;
#pragma unroll
        for (int u = 0; u < KPW; ++u) {
          const unsigned off = ok ? (unsigned)(((tile * ksteps + w * KPW + u) * 64 + lane) * 16) : MG_OOB;
          wa[j][u] = buf_load16_stream(rg, off);
          wb[j][u] = buf_load16_stream(ru, off);
        }
      };
      load_glu(0, gt0);
      load_glu(1, gt0 + 1);
      {
        const bool bad = poll(a.xbuf[xsel], nxw, tag_x, xw, std::integral_constant<int, NXW>());
        MG_CHECK(bad);
        have_x = true;
      }
      norm_rows(L.mlp_norm_w);
      uint4 xb[KPW];
      load_xb(xb);
      for (int t0 = gt0; t0 < gt1; t0 += 2) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          floatx4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int u = 0; u < KPW; ++u) {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[j][u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
            acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb[j][u]), as_bf16x8(xb[u]), acc2, 0, 0, 0);
          }
          stash(2 * j, acc);
          stash(2 * j + 1, acc2);
          load_glu(j, t0 + 2 + j);
        }
        __syncthreads();
        if (w < 2 && t0 + w < gt1) {
          float og[4], ou[4];
          reduce_slot(2 * w, og);
          reduce_slot(2 * w + 1, ou);
          const int tile = t0 + w;
          const int half = 2 * tile + (g >> 1);
          if (xrow && half >= h0 && half < h1) {
            float o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = rnd_bf16(gelu_tanh_fast(rnd_bf16(og[i]))) * rnd_bf16(ou[i]);
            u64* dst = a.act + (((size_t)r * I + tile * 16 + 4 * g) >> 1);
            st_agent(dst, ((u64)tag_act << 32) | pack2_bf16(o[0], o[1]));
            st_agent(dst + 1, ((u64)tag_act << 32) | pack2_bf16(o[2], o[3]));
          }
        }
        __syncthreads();
      }
    }

    // ============================================================== S3: down projection, (tile group, K chunk)
    MG_PHASE();
    const unsigned tag_part = tbase | (++ph);
    if (wg < ntg * KS) {
      const int dt0 = dgrp * tpg, dt1 = min(tiles_d, dt0 + tpg);
      const rsrc_t rd = make_rsrc(L.wp_down, (size_t)tiles_d * kst_I * 1024);
      uint4 wd[MG_NBD][MG_KD];
      auto load_down = [&](int j, int tile) {
#pragma unroll
        for (int u = 0; u < MG_KD; ++u) {
          const int ks = w + 8 * u;
          wd[j][u] = buf_load16_stream(rd, (tile < dt1 && ks < kch) ? (unsigned)(((tile * kst_I + dchunk * kch + ks) * 64 + lane) * 16) : MG_OOB);
        }
      };
#pragma unroll
      for (int j = 0; j < MG_NBD; ++j) load_down(j, dt0 + j);
      // this lane's activation fragments straight from the tagged words: row r, columns 32*ks + 8*g .. +8
      uint4 xb[MG_KD];
      {
        u64 v[MG_KD][4];
        int spins = 0;
        bool bad = false;
        {
          // probe with one word per lane and a pause (see poll)
          const u64* src = a.act + (((size_t)(xrow ? r : 0) * I + (size_t)(dchunk * kch + w) * 32 + g * 8) >> 1);
          const bool mine = xrow && w < kch;
          for (;;) {
            const u64 p0 = mine ? ld_agent(src) : ((u64)tag_act << 32);
            if ((unsigned)(p0 >> 32) == tag_act) break;
            if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
            __builtin_amdgcn_s_sleep(2);
          }
        }
        for (; !bad;) {
          bool ok = true;
#pragma unroll
          for (int u = 0; u < MG_KD; ++u) {
            const int ks = w + 8 * u;
            const u64* src = a.act + (((size_t)(xrow ? r : 0) * I + (size_t)(dchunk * kch + ks) * 32 + g * 8) >> 1);
#pragma unroll
            for (int q = 0; q < 4; ++q) v[u][q] = (xrow && ks < kch) ? ld_agent(src + q) : ((u64)tag_act << 32);
          }
#pragma unroll
          for (int u = 0; u < MG_KD; ++u)
#pragma unroll
            for (int q = 0; q < 4; ++q) ok = ok && (unsigned)(v[u][q] >> 32) == tag_act;
          if (ok) break;
          if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
        }
#pragma unroll
        for (int u = 0; u < MG_KD; ++u) xb[u] = make_uint4((unsigned)v[u][0], (unsigned)v[u][1], (unsigned)v[u][2], (unsigned)v[u][3]);
        MG_CHECK(bad);
      }
      for (int t0 = dt0; t0 < dt1; t0 += MG_NBD) {
#pragma unroll
        for (int j = 0; j < MG_NBD; ++j) {
          floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int u = 0; u < MG_KD; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wd[j][u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
          stash(j, acc);
          load_down(j, t0 + MG_NBD + j);
        }
        __syncthreads();
        if (w < MG_NBD && t0 + w < dt1) {
          float o[4];
          reduce_slot(w, o);
          if (xrow) {
            u64* dst = a.part + ((size_t)dchunk * B + r) * d + (t0 + w) * 16 + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; ++i) st_agent(dst + i, ((u64)tag_part << 32) | __float_as_uint(o[i]));
          }
        }
        __syncthreads();
      }
    }

    // ============================================================== S4: K chunks summed in order + residual, tile `wg`
    MG_PHASE();
    const unsigned tag_out2 = tbase | (++ph);
    if (wg < tiles_d) {
      // thread (row, column pair) sums its KS chunks
      const int npair = B * 8;
      float s0 = 0.f, s1 = 0.f;
      bool bad = false;
      if (tid < npair) {
        const int row = tid >> 3, cp = tid & 7;
        const u64* src = a.part + (size_t)row * d + wg * 16 + 2 * cp;
        for (int c0 = 0; c0 < KS; c0 += 8) {
          u64 v[8][2];
          int spins = 0;
          for (;;) {
            bool ok = true;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              const bool in = c0 + k < KS;
              v[k][0] = in ? ld_agent(src + (size_t)(c0 + k) * B * d) : ((u64)tag_part << 32);
              v[k][1] = in ? ld_agent(src + (size_t)(c0 + k) * B * d + 1) : ((u64)tag_part << 32);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) ok = ok && (unsigned)(v[k][0] >> 32) == tag_part && (unsigned)(v[k][1] >> 32) == tag_part;
            if (ok) break;
            if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
            __builtin_amdgcn_s_sleep(2);
          }
#pragma unroll
          for (int k = 0; k < 8; ++k) { s0 += __uint_as_float((unsigned)v[k][0]); s1 += __uint_as_float((unsigned)v[k][1]); }
          if (bad) break;
        }
        if (!bad) {
          const float* xr = xt + row * 16 + 2 * cp;
          // xt holds x' of this tile (kept by the gate/up phase's norm)
          st_agent(a.xbuf[xsel ^ 1] + (((size_t)row * d + wg * 16 + 2 * cp) >> 1),
                   ((u64)tag_out2 << 32) | pack2_bf16(xr[0] + rnd_bf16(s0), xr[1] + rnd_bf16(s1)));
        }
      }
      MG_CHECK(bad);
    }
    xsel ^= 1;
    tag_x = tag_out2;
    have_x = false;
  }

  // ================================================================ F1: final norm, tied head, row maxima
  MG_PHASE();
  const unsigned tag_best = tbase | (++ph);
  {
    const int tiles_v = (a.V + 15) >> 4;
    const int vt0 = (int)(((long long)wg * tiles_v) / G), vt1 = (int)(((long long)(wg + 1) * tiles_v) / G);
    const rsrc_t rw = make_rsrc(a.wp_emb, (size_t)tiles_v * ksteps * 1024);
    uint4 wa[MG_NB][KPW];
    auto load_head = [&](int j, int tile) {
#pragma unroll
      for (int u = 0; u < KPW; ++u)
        wa[j][u] = buf_load16_stream(rw, tile < vt1 ? (unsigned)(((tile * ksteps + w * KPW + u) * 64 + lane) * 16) : MG_OOB);
    };
#pragma unroll
    for (int j = 0; j < MG_NB; ++j) load_head(j, vt0 + j);
    if (!have_x) {
      const bool bad = poll(a.xbuf[xsel], nxw, tag_x, xw, std::integral_constant<int, NXW>());
      MG_CHECK(bad);
    }
    norm_rows(a.final_norm_w);
    uint4 xb[KPW];
    load_xb(xb);
    u64 bestk = 0ull;
    for (int t0 = vt0; t0 < vt1; t0 += MG_NB) {
#pragma unroll
      for (int j = 0; j < MG_NB; ++j) {
        floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KPW; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[j][u]), as_bf16x8(xb[u]), acc, 0, 0, 0);
        stash(j, acc);
        load_head(j, t0 + MG_NB + j);
      }
      __syncthreads();
      if (w < MG_NB && t0 + w < vt1) {
        float o[4];
        reduce_slot(w, o);
        if (xrow) {
          const int f0 = (t0 + w) * 16 + 4 * g;
          bf16_t* dst = a.logits + (size_t)r * a.V + f0;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (f0 + i < a.V) {
              const bf16_t lb = f32_to_bf16(o[i]);
              dst[i] = lb;
              float lv = bf16_to_f32(lb);
              if (a.temperature != 1.0f) lv = rnd_bf16(lv / a.temperature);
              lv = rnd_bf16(fminf(fmaxf(lv, -1e4f), 1e4f));
              const u64 k = ((u64)f32_okey(lv) << 32) | (u64)(0xffffffffu - (unsigned)(f0 + i));
              bestk = k > bestk ? k : bestk;
            }
          }
        }
      }
      __syncthreads();
    }
    if (a.greedy) {
      // best of the workgroup per batch row: across the 4 feature groups of a lane row, then across the reducing waves
      u64 o = __shfl_xor(bestk, 16, 64);
      bestk = o > bestk ? o : bestk;
      o = __shfl_xor(bestk, 32, 64);
      bestk = o > bestk ? o : bestk;
      u64* bw = (u64*)red;
      if (w < MG_NB && g == 0) bw[w * 16 + r] = bestk;
      __syncthreads();
      if (tid < B) {
        u64 k = bw[tid];
#pragma unroll
        for (int j = 1; j < MG_NB; ++j) k = bw[j * 16 + tid] > k ? bw[j * 16 + tid] : k;
        // two tagged words per (workgroup, row): value key, index
        u64* dst = a.best + ((size_t)wg * 16 + tid) * 2;
        st_agent(dst, ((u64)tag_best << 32) | (unsigned)(k >> 32));
        st_agent(dst + 1, ((u64)tag_best << 32) | (unsigned)k);
      }
    }
  }

  // ================================================================ F2: greedy token, counters
  MG_PHASE();
  if (wg == 0) {
    bool bad = false;
    if (a.greedy) {
      // wave w takes rows w, w+8: each lane polls G/64 workgroups' words of that row
      for (int row = w; row < B; row += 8) {
        u64 bk = 0ull;
        for (int g0 = lane; g0 < G; g0 += 64) {
          const u64* src = a.best + ((size_t)g0 * 16 + row) * 2;
          u64 v0, v1;
          int spins = 0;
          for (;;) {
            v0 = ld_agent(src);
            v1 = ld_agent(src + 1);
            if ((unsigned)(v0 >> 32) == tag_best && (unsigned)(v1 >> 32) == tag_best) break;
            if (++spins > MG_SPIN_LIMIT || ((spins & 31) == 0 && ld_agent32(a.ctrl + MG_CTRL_ABORT) != 0u)) { bad = true; break; }
            __builtin_amdgcn_s_sleep(2);
          }
          const u64 k = ((u64)(unsigned)v0 << 32) | (unsigned)v1;
          bk = k > bk ? k : bk;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          const u64 t = __shfl_xor(bk, o, 64);
          bk = t > bk ? t : bk;
        }
        if (lane == 0 && !bad) a.tok_out[(size_t)row * a.tok_stride + pos] = (int64_t)(0xffffffffu - (unsigned)(bk & 0xffffffffull));
      }
    }
    MG_CHECK(bad);
    if (tid == 0) {
      a.ctrl[MG_CTRL_EPOCH] = epoch + 1;
      if (a.dyn && a.greedy) { a.dyn[0] = pos + 1; a.dyn[1] += 1; }
    }
  }
#undef MG_CHECK
#undef MG_PHASE
}

struct MegaPlan {
  int G, KS, kpw, nxw;
  size_t off_layers, off_x0, off_x1, off_qkv, off_att, off_act, off_part, off_best, bytes, shm;
};

int query_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    else cus = 256;
  }
  return cus;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Returns false when the shape is not covered.
bool mega_plan(const fstu_model_desc* m, MegaPlan* p) {
  if (!m || m->dtype != FSTU_BF16 || m->stu_mode != 1 || m->single_branch) return false;
  const int B = m->B, d = m->d, I = m->I;
  if (B < 1 || B > 16 || d % 256 != 0 || d > 4096 || I % 32 != 0 || m->V < 16) return false;
  if (m->head_dim != 64 && m->head_dim != 128) return false;
  if (m->n_heads * m->head_dim != d || m->lds_S < 1 || m->n_layers > 40) return false;
  const int G = query_cus();
  if (G < 64 || G % 16 != 0) return false;
  const int KS = 16;
  const int kst_I = I / 32;
  if (kst_I % KS != 0 || (kst_I / KS + 7) / 8 > MG_KD) return false;
  const int kpw = d / 256;
  if (kpw != 3 && kpw != 4 && kpw != 8) return false;
  const int words = B * d / 2;
  const int nxw = (words + MG_THREADS - 1) / MG_THREADS;
  if (nxw > 32) return false;
  if (m->kv_cap + 1 > 2048) return false;                                        // attention scores live in 2048 floats of LDS
  if ((MG_THREADS / (m->head_dim / 8)) * m->head_dim > MG_NB * 8 * 256 - 2048) return false;
  if (3 * m->head_dim > 384) return false;
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    if (!L.wp_gate || !L.wp_up || !L.wp_down || !L.norm1_w || !L.mlp_norm_w) return false;
    // (the one-launch step does not carry the exact head of the filter)
    if (L.kind == 0) { if (!L.wp_m_inputs || !L.lds_state || !L.lds_a || !L.lds_ce || !L.lds_co || L.lds_fir) return false; }
    else if (!L.wp_qkv || !L.wp_proj || !L.kring || !L.vring || !L.slopes) return false;
  }
  if (!m->wp_emb || !m->emb || !m->final_norm_w || !m->logits) return false;
  p->G = G; p->KS = KS; p->kpw = kpw; p->nxw = nxw;
  size_t off = 1024;                                  // control words
  p->off_layers = off; off = align_up(off + sizeof(MegaLayer) * (size_t)m->n_layers, 256);
  p->off_x0 = off; off = align_up(off + (size_t)words * 8, 256);
  p->off_x1 = off; off = align_up(off + (size_t)words * 8, 256);
  p->off_qkv = off; off = align_up(off + (size_t)words * 3 * 8, 256);
  p->off_att = off; off = align_up(off + (size_t)words * 8, 256);
  p->off_act = off; off = align_up(off + (size_t)B * I / 2 * 8, 256);
  p->off_part = off; off = align_up(off + (size_t)KS * B * d * 8, 256);
  p->off_best = off; off = align_up(off + (size_t)G * 16 * 2 * 8, 256);
  p->bytes = off;
  p->shm = align_up((size_t)B * (d + 8) * 2, 16) + (size_t)(MG_NB * 8 * 256 + 256 + 256 + 256 + 512) * 4;
  return p->shm <= 150 * 1024;
}

}  // namespace

extern "C" size_t fstu_step_mega_ws_bytes(const fstu_model_desc* m) {
  MegaPlan p;
  return mega_plan(m, &p) ? p.bytes : 0;
}

extern "C" int fstu_step_mega_prepare(const fstu_model_desc* m, void* ws, void* stream) {
  MegaPlan p;
  FSTU_REQUIRE(m && ws, FSTU_ENULL, "fstu_step_mega_prepare: null pointer");
  FSTU_REQUIRE(mega_plan(m, &p), FSTU_ESHAPE, "fstu_step_mega_prepare: this model is not covered by the one-launch step");
  FSTU_REQUIRE(fstu_aligned(ws, 256), FSTU_EALIGN, "fstu_step_mega_prepare: workspace must be 256-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = hipMemsetAsync(ws, 0, p.bytes, s);
  if (e != hipSuccess) { fstu_set_error("fstu_step_mega_prepare: memset: %s", hipGetErrorString(e)); return (int)e; }
  std::vector<MegaLayer> tab((size_t)m->n_layers);
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    MegaLayer& t = tab[l];
    t.kind = L.kind; t.pad = 0;
    t.norm1_w = (const bf16_t*)L.norm1_w; t.mlp_norm_w = (const bf16_t*)L.mlp_norm_w;
    t.wp_first = (const uint4*)(L.kind == 0 ? L.wp_m_inputs : L.wp_qkv);
    t.wp_proj = (const uint4*)L.wp_proj;
    t.wp_gate = (const uint4*)L.wp_gate; t.wp_up = (const uint4*)L.wp_up; t.wp_down = (const uint4*)L.wp_down;
    t.state = L.lds_state; t.a = L.lds_a; t.ce = L.lds_ce; t.co = L.lds_co;
    t.kring = (bf16_t*)L.kring; t.vring = (bf16_t*)L.vring; t.slopes = L.slopes;
  }
  // pageable host memory: the copy is complete (staged) when the call returns
  e = hipMemcpyAsync((char*)ws + p.off_layers, tab.data(), sizeof(MegaLayer) * tab.size(), hipMemcpyHostToDevice, s);
  if (e != hipSuccess) { fstu_set_error("fstu_step_mega_prepare: copy: %s", hipGetErrorString(e)); return (int)e; }
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) { fstu_set_error("fstu_step_mega_prepare: sync: %s", hipGetErrorString(e)); return (int)e; }
  return FSTU_OK;
}

extern "C" int fstu_step_mega_status(const void* ws, int* err_out) {
  FSTU_REQUIRE(ws && err_out, FSTU_ENULL, "fstu_step_mega_status: null pointer");
  unsigned v = 0;
  hipError_t e = hipMemcpy(&v, (const char*)ws + MG_CTRL_ERR * 4, 4, hipMemcpyDeviceToHost);
  if (e != hipSuccess) { fstu_set_error("fstu_step_mega_status: %s", hipGetErrorString(e)); return (int)e; }
  *err_out = (int)v;
  return FSTU_OK;
}

template <int KPW, int NXW>
static int mega_launch_t(const MegaArgs& a, const MegaPlan& p, hipStream_t s) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&]() {
    attr_err = hipFuncSetAttribute((const void*)mega_step_kernel<KPW, NXW>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
  });
  if (attr_err != hipSuccess) { fstu_set_error("fstu_step_mega: hipFuncSetAttribute: %s", hipGetErrorString(attr_err)); return (int)attr_err; }
  int per_cu = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mega_step_kernel<KPW, NXW>, MG_THREADS, p.shm);
  if (e != hipSuccess || per_cu < 1) { fstu_set_error("fstu_step_mega: the kernel does not fit a compute unit (%d)", per_cu); return FSTU_ESHAPE; }
  hipLaunchKernelGGL((mega_step_kernel<KPW, NXW>), dim3(p.G), dim3(MG_THREADS), p.shm, s, a);
  FSTU_CHECK_LAUNCH("fstu_step_mega");
  return FSTU_OK;
}

// tokens: column 0 of the token buffer; the step reads column pos and (greedy) writes column pos+1.
int fstu_step_mega_launch(const fstu_model_desc* m, int64_t* tokens, int64_t* tok_out, int64_t tok_stride, int pos,
                          float temperature, int greedy, int* dyn, void* stream) {
  MegaPlan p;
  FSTU_REQUIRE(m && m->mega_ws && tokens, FSTU_ENULL, "fstu_step_mega: null pointer");
  FSTU_REQUIRE(mega_plan(m, &p), FSTU_ESHAPE, "fstu_step_mega: this model is not covered by the one-launch step");
  FSTU_REQUIRE(temperature > 0.f && tok_stride >= 1 && pos >= 0, FSTU_EARG, "fstu_step_mega: bad temperature / stride / position");
  char* ws = (char*)m->mega_ws;
  MegaArgs a;
  a.layers = (const MegaLayer*)(ws + p.off_layers);
  a.emb = (const bf16_t*)m->emb; a.wp_emb = (const uint4*)m->wp_emb; a.final_norm_w = (const bf16_t*)m->final_norm_w;
  a.xbuf[0] = (u64*)(ws + p.off_x0); a.xbuf[1] = (u64*)(ws + p.off_x1);
  a.qkv = (u64*)(ws + p.off_qkv); a.att = (u64*)(ws + p.off_att); a.act = (u64*)(ws + p.off_act);
  a.part = (u64*)(ws + p.off_part); a.best = (u64*)(ws + p.off_best);
  a.ctrl = (unsigned*)ws; a.logits = (bf16_t*)m->logits; a.tokens = tokens; a.tok_out = tok_out; a.dyn = dyn; a.tok_stride = tok_stride;
  a.n_layers = m->n_layers; a.B = m->B; a.d = m->d; a.I = m->I; a.V = m->V; a.H = m->n_heads; a.hd = m->head_dim;
  a.window = m->window; a.cap = m->kv_cap; a.S = m->lds_S; a.pos = pos; a.greedy = greedy; a.ks_down = p.KS;
  a.eps = m->eps; a.softcap = m->softcap; a.temperature = temperature;
  hipStream_t s = (hipStream_t)stream;
#define MG_CASE(K, N) if (p.kpw == K && p.nxw <= N) return mega_launch_t<K, N>(a, p, s)
  MG_CASE(3, 6);
  MG_CASE(3, 12);
  MG_CASE(4, 16);
  MG_CASE(8, 16);
  MG_CASE(8, 32);
#undef MG_CASE
  fstu_set_error("fstu_step_mega: no kernel for d=%d B=%d", m->d, m->B);
  return FSTU_ESHAPE;
}

bool fstu_step_mega_ok(const fstu_model_desc* m) {
  MegaPlan p;
  return m && m->mega_ws && mega_plan(m, &p);
}
