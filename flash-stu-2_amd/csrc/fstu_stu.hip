// STU kernels: per-token decode step in the exact history form and in the
// distilled diagonal-recurrence (LDS) form, the state builder that turns a
// prefilled history into recurrence state, the time-domain prefill
// convolution, and the dense LDS step of mini_stu.
#include "fstu_common.h"
#include "fstu_prologue.h"

// ---------------------------------------------------------------- history step
// Lags are rows of the (lag, channel) plane; a workgroup walks a contiguous
// lag range with all loads coalesced along channels.  Thread (row, chunk)
// accumulates VEC channels for lags row, row+RW, ...; rows are then reduced
// through LDS.  Even and odd lags are kept apart because the reference rounds
// the two sign branches separately.
template <typename T, int VEC>
struct VecLd;
template <> struct VecLd<bf16_t, 8> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float* o) {
    uint4 v = *(const uint4*)p;
    unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <> struct VecLd<float, 8> {
  static __device__ __forceinline__ void ld(const float* p, float* o) {
    float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};
template <typename T> struct VecLd<T, 1> {
  static __device__ __forceinline__ void ld(const T* p, float* o) { o[0] = DT<T>::ld(p); }
};

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
stu_step_hist_kernel(const T* __restrict__ hist, const T* __restrict__ filt, float* __restrict__ eo, int B, int d,
                     int t, int cap, int nl, int per, int CW, int RW) {
  __shared__ float sh[256 * 2 * VEC];
  const int b = blockIdx.y, split = blockIdx.x;
  const int nch = d / VEC;
  const int chunk = blockIdx.z * CW + (threadIdx.x % CW);
  const int row = threadIdx.x / CW;
  const bool active = row < RW && chunk < nch;
  float aE[VEC], aO[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { aE[v] = 0.f; aO[v] = 0.f; }
  const int lag0 = split * per, lag1 = min(nl, lag0 + per);
  if (active) {
    const T* hb = hist + ((size_t)b * cap + t) * d + (size_t)chunk * VEC;
    const T* fb = filt + (size_t)chunk * VEC;
#pragma unroll 4
    for (int lag = lag0 + row; lag < lag1; lag += RW) {
      float h[VEC], f[VEC];
      VecLd<T, VEC>::ld(hb - (size_t)lag * d, h);
      VecLd<T, VEC>::ld(fb + (size_t)lag * d, f);
      if (lag & 1) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) aO[v] = fmaf(f[v], h[v], aO[v]);
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) aE[v] = fmaf(f[v], h[v], aE[v]);
      }
    }
  }
  float* mine = sh + (size_t)threadIdx.x * 2 * VEC;
#pragma unroll
  for (int v = 0; v < VEC; ++v) { mine[v] = aE[v]; mine[VEC + v] = aO[v]; }
  __syncthreads();
  if (active && row == 0) {
    for (int r2 = 1; r2 < RW; ++r2) {
      const float* o = sh + (size_t)(r2 * CW + (threadIdx.x % CW)) * 2 * VEC;
#pragma unroll
      for (int v = 0; v < VEC; ++v) { aE[v] += o[v]; aO[v] += o[VEC + v]; }
    }
    float* pe = eo + ((size_t)(2 * split) * B + b) * d + (size_t)chunk * VEC;
    float* po = eo + ((size_t)(2 * split + 1) * B + b) * d + (size_t)chunk * VEC;
#pragma unroll
    for (int v = 0; v < VEC; ++v) { pe[v] = aE[v]; po[v] = aO[v]; }
  }
}

extern "C" int fstu_stu_step_hist(const void* hist, const void* filt, float* eo, int B, int d, int t, int cap, int L,
                                  int nsplit, int dtype, void* stream) {
  FSTU_REQUIRE(hist && filt && eo, FSTU_ENULL, "fstu_stu_step_hist: null pointer");
  FSTU_REQUIRE(B >= 1 && d >= 1 && L >= 1 && cap >= 1, FSTU_ESHAPE, "fstu_stu_step_hist: bad shape B=%d d=%d L=%d cap=%d", B, d, L, cap);
  FSTU_REQUIRE(t >= 0 && t < cap, FSTU_EARG, "fstu_stu_step_hist: t=%d outside history capacity %d", t, cap);
  FSTU_REQUIRE(nsplit >= 1 && nsplit <= 4096, FSTU_EARG, "fstu_stu_step_hist: nsplit=%d", nsplit);
  const int nl = (t + 1 < L) ? t + 1 : L;
  const int per = (nl + nsplit - 1) / nsplit;
  const bool vec8 = (d % 8 == 0) && fstu_aligned(hist, 16) && fstu_aligned(filt, 16);
  const int nch = vec8 ? d / 8 : d;
  const int CW = nch < 256 ? nch : 256;
  const int RW = 256 / CW;
  dim3 grid(nsplit, B, (nch + CW - 1) / CW);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == FSTU_BF16) {
    if (vec8) hipLaunchKernelGGL((stu_step_hist_kernel<bf16_t, 8>), grid, dim3(256), 0, s, (const bf16_t*)hist, (const bf16_t*)filt, eo, B, d, t, cap, nl, per, CW, RW);
    else hipLaunchKernelGGL((stu_step_hist_kernel<bf16_t, 1>), grid, dim3(256), 0, s, (const bf16_t*)hist, (const bf16_t*)filt, eo, B, d, t, cap, nl, per, CW, RW);
  } else if (dtype == FSTU_F32) {
    if (vec8) hipLaunchKernelGGL((stu_step_hist_kernel<float, 8>), grid, dim3(256), 0, s, (const float*)hist, (const float*)filt, eo, B, d, t, cap, nl, per, CW, RW);
    else hipLaunchKernelGGL((stu_step_hist_kernel<float, 1>), grid, dim3(256), 0, s, (const float*)hist, (const float*)filt, eo, B, d, t, cap, nl, per, CW, RW);
  } else {
    fstu_set_error("fstu_stu_step_hist: unknown dtype %d", dtype);
    return FSTU_EDTYPE;
  }
  FSTU_CHECK_LAUNCH("fstu_stu_step_hist");
  return FSTU_OK;
}

// ---------------------------------------------------------------- exact head of the distilled filter
// The recurrence reproduces the effective filter phi_proj up to its lag-by-lag bf16 rounding, which is largest on the
// first lags.  fir[s, c] = f[s, c] - f_fit[s, c] for the first R lags (R a power of two, a multiple of 8) corrects them
// exactly from a ring of the last R projected inputs (ring[b, p % R, c] = x_proj of position p, zero before the first
// position): even lags add to E, odd lags to O.  Mode group g of a (row, 4 channels) pair takes lags g, g+8, ...: their
// parity is that of g, so the partial sum joins E (g even) or O (g odd) before the reduction over the mode groups.
template <typename T> struct Ring4 {
  static __device__ __forceinline__ void ld(const T* p, float (&v)[4]) {
    const float4 q = *(const float4*)p;
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
  static __device__ __forceinline__ void st(T* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Ring4<bf16_t> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float (&v)[4]) {
    const uint2 q = *(const uint2*)p;
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float (&v)[4]) {
    *(uint2*)p = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
  }
};
// ---------------------------------------------------------------- LDS-form step
// Workgroup = 32 channel quads (128 channels) x 8 mode groups.  Each thread
// advances S/8 modes of 4 channels (float4 state accesses, 512 contiguous
// bytes per mode row and wave half), then the 8 mode groups are reduced in LDS.
//
// omode (with co and ocache (B,d) fp32): the odd-lag sum O of a step weighs the bank the PREVIOUS step advanced, which
// nothing has touched since, and the odd lags of the exact head reach the inputs the previous step already held.  So
// a step can form the next step's O while it has its own bank in registers and leave it in ocache:
//   omode 1  O of this step comes from ocache; the next step's O is formed on this bank after its advance (the same
//            products in the same order as the plain step would form them one step later: bit-identical) and stored.
//            The other bank is not read: a third less state traffic.
//   omode 2  priming for position t (the last position of a prompt): nothing is advanced and nothing is written but
//            ocache, which receives what a step at position t would have left for position t+1; x is taken from the
//            ring (or not at all without the exact head).
#define LDS_JG 8
// state rows of the wide step: read once and written once per two steps, far more than the caches hold in between
typedef float f32x4_nt __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld_state_nt(const float* p) {
  const f32x4_nt v = __builtin_nontemporal_load((const f32x4_nt*)p);
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st_state_nt(float* p, float4 h) {
  const f32x4_nt v = {h.x, h.y, h.z, h.w};
  __builtin_nontemporal_store(v, (f32x4_nt*)p);
}
// (OM: the mode as a template parameter, so that each instance holds only the operands its mode requests)
template <typename T, int OM>
__global__ void __launch_bounds__(256)
stu_step_lds_kernel(float* __restrict__ state, const T* __restrict__ xp, int ldxp, const float* __restrict__ a,
                    const float* __restrict__ ce, const float* __restrict__ co /*optional: weights of the other bank*/,
                    float scale, T* __restrict__ y, int ldy, int S, int d, int parity, const int* __restrict__ dyn,
                    int pair /* != 0 (needs co): y = T(T(E+O) + T(E-O)), the two sign branches rounded separately */,
                    T* __restrict__ ring /*optional (B,R,d), with fir (R,d) and co: exact head of the filter*/,
                    const float* __restrict__ fir, int R, int t, const int* __restrict__ pos_dyn,
                    const T* res /*optional, rows of stride ldy: y = T(res + T(output)); may be y itself*/,
                    float* ocache) {
  constexpr int omode = OM;
  __shared__ float sh[LDS_JG][32][4];
  __shared__ float sho[LDS_JG][32][4];
  __shared__ float shf[LDS_JG][32][4];   // omode: the exact head's share of the next step's O, in the odd slots
  if (dyn) parity = dyn[0] & 1;
  if (pos_dyn) t = pos_dyn[0];
  const int b = blockIdx.y;
  const int q = threadIdx.x & 31, jg = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + q) * 4;
  const bool ok = c < d;
  const bool head = co && fir;
  constexpr bool prime = OM == 2;
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, acco[4] = {0.f, 0.f, 0.f, 0.f}, fnx[4] = {0.f, 0.f, 0.f, 0.f};
  float rsd[4] = {0.f, 0.f, 0.f, 0.f}, ocur[4] = {0.f, 0.f, 0.f, 0.f};
  if (ok) {
    // the residual row piece the epilogue adds and the cached O: the oldest requests, so no wait for a later one
    // depends on these branches
    if (res) Ring4<T>::ld(res + (size_t)b * ldy + c, rsd);
    if constexpr (OM == 1) Ring4<float>::ld(ocache + (size_t)b * d + c, ocur);
    // Every operand of the thread's first 8 modes of both banks and first 8 lags of the head goes in flight before
    // anything waits (out-of-range modes and lags re-read a valid element and are ignored): one trip to memory for
    // S <= 64 and 64 taps; longer states and heads continue in loops.
    constexpr int PJ = 8;
    float* st = state + (((size_t)b * 2 + parity) * S) * d + c;
    const float* so = state + (((size_t)b * 2 + (parity ^ 1)) * S) * d + c;
    const T* rb = head ? ring + (size_t)b * R * d + c : nullptr;
    // omode: only the even mode groups take lags (the even ones, for this step's E and, shifted by one, the next O)
    const bool lags = head && (omode == 0 || (jg & 1) == 0);
    float4 ph[PJ], pc[PJ], qh[PJ], qc[PJ], fr[PJ], fr2[PJ];
    float pa[PJ], rx[PJ][4];
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int j = min(jg + LDS_JG * k, S - 1);
      ph[k] = OM == 1 ? ld_state_nt(st + (size_t)j * d) : *(const float4*)(st + (size_t)j * d);
      pc[k] = *(const float4*)(ce + (size_t)j * d + c);
      pa[k] = a[j];
    }
    if (co) {
#pragma unroll
      for (int k = 0; k < PJ; ++k) {
        const int j = min(jg + LDS_JG * k, S - 1);
        if constexpr (OM == 0) qh[k] = *(const float4*)(so + (size_t)j * d);
        qc[k] = *(const float4*)(co + (size_t)j * d + c);
      }
    }
    if (lags) {
#pragma unroll
      for (int k = 0; k < PJ; ++k) {
        const int sl = min(jg + 8 * k, R - 1);
        Ring4<T>::ld(rb + (size_t)((t - sl) & (R - 1)) * d, rx[k]);
        fr[k] = *(const float4*)(fir + (size_t)sl * d + c);
        if constexpr (OM != 0) fr2[k] = *(const float4*)(fir + (size_t)min(sl + 1, R - 1) * d + c);
      }
    }
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (!prime) {
#pragma unroll
      for (int v = 0; v < 4; ++v) x[v] = DT<T>::ld(xp + (size_t)b * ldxp + c + v);
    } else if (head) {
      Ring4<T>::ld(rb + (size_t)(t & (R - 1)) * d, x);
    }
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int j = jg + LDS_JG * k;
      if (j < S) {
        float4 h = ph[k];
        if constexpr (!prime) {
          h.x = fmaf(pa[k], h.x, x[0]);
          h.y = fmaf(pa[k], h.y, x[1]);
          h.z = fmaf(pa[k], h.z, x[2]);
          h.w = fmaf(pa[k], h.w, x[3]);
          if constexpr (OM == 1) st_state_nt(st + (size_t)j * d, h); else *(float4*)(st + (size_t)j * d) = h;
          acc[0] = fmaf(pc[k].x, h.x, acc[0]);
          acc[1] = fmaf(pc[k].y, h.y, acc[1]);
          acc[2] = fmaf(pc[k].z, h.z, acc[2]);
          acc[3] = fmaf(pc[k].w, h.w, acc[3]);
        }
        if constexpr (OM != 0) {   // the next step's odd-lag sum on this bank
          acco[0] = fmaf(qc[k].x, h.x, acco[0]);
          acco[1] = fmaf(qc[k].y, h.y, acco[1]);
          acco[2] = fmaf(qc[k].z, h.z, acco[2]);
          acco[3] = fmaf(qc[k].w, h.w, acco[3]);
        }
      }
    }
#pragma unroll 4
    for (int j = jg + LDS_JG * PJ; j < S; j += LDS_JG) {
      float4 h = *(float4*)(st + (size_t)j * d);
      if constexpr (!prime) {
        const float4 cj = *(const float4*)(ce + (size_t)j * d + c);
        const float aj = a[j];
        h.x = fmaf(aj, h.x, x[0]);
        h.y = fmaf(aj, h.y, x[1]);
        h.z = fmaf(aj, h.z, x[2]);
        h.w = fmaf(aj, h.w, x[3]);
        *(float4*)(st + (size_t)j * d) = h;
        acc[0] = fmaf(cj.x, h.x, acc[0]);
        acc[1] = fmaf(cj.y, h.y, acc[1]);
        acc[2] = fmaf(cj.z, h.z, acc[2]);
        acc[3] = fmaf(cj.w, h.w, acc[3]);
      }
      if constexpr (OM != 0) {
        const float4 oj = *(const float4*)(co + (size_t)j * d + c);
        acco[0] = fmaf(oj.x, h.x, acco[0]);
        acco[1] = fmaf(oj.y, h.y, acco[1]);
        acco[2] = fmaf(oj.z, h.z, acco[2]);
        acco[3] = fmaf(oj.w, h.w, acco[3]);
      }
    }
    if (co) {
      if constexpr (OM == 0) {
        // odd lags: lag 2m+1 reaches position t-1-2m, which the bank of the other parity holds (not advanced here)
#pragma unroll
        for (int k = 0; k < PJ; ++k) {
          if (jg + LDS_JG * k < S) {
            acco[0] = fmaf(qc[k].x, qh[k].x, acco[0]);
            acco[1] = fmaf(qc[k].y, qh[k].y, acco[1]);
            acco[2] = fmaf(qc[k].z, qh[k].z, acco[2]);
            acco[3] = fmaf(qc[k].w, qh[k].w, acco[3]);
          }
        }
#pragma unroll 4
        for (int j = jg + LDS_JG * PJ; j < S; j += LDS_JG) {
          const float4 h = *(const float4*)(so + (size_t)j * d);
          const float4 oj = *(const float4*)(co + (size_t)j * d + c);
          acco[0] = fmaf(oj.x, h.x, acco[0]);
          acco[1] = fmaf(oj.y, h.y, acco[1]);
          acco[2] = fmaf(oj.z, h.z, acco[2]);
          acco[3] = fmaf(oj.w, h.w, acco[3]);
        }
      }
      if (lags) {
        // exact head: lags jg, jg+8, ... share the parity of jg; a position before the sequence contributes nothing.
        // omode: the same inputs, weighted with the next lag's taps, are the odd lags of the next step (lag sl+1 of
        // position t+1 is lag sl of position t), summed in the order the plain step uses for its odd mode groups.
        float f[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < PJ; ++k) {
          const int sl = jg + 8 * k;
          if (sl < R) {
            const float m = (t - sl >= 0) ? 1.f : 0.f;
            float xv[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) xv[v] = sl == 0 ? x[v] : m * rx[k][v];
            if constexpr (!prime) {
              f[0] = fmaf(fr[k].x, xv[0], f[0]);
              f[1] = fmaf(fr[k].y, xv[1], f[1]);
              f[2] = fmaf(fr[k].z, xv[2], f[2]);
              f[3] = fmaf(fr[k].w, xv[3], f[3]);
            }
            if (OM != 0 && sl + 1 < R) {
              fnx[0] = fmaf(fr2[k].x, xv[0], fnx[0]);
              fnx[1] = fmaf(fr2[k].y, xv[1], fnx[1]);
              fnx[2] = fmaf(fr2[k].z, xv[2], fnx[2]);
              fnx[3] = fmaf(fr2[k].w, xv[3], fnx[3]);
            }
          }
        }
#pragma unroll 4
        for (int sl = jg + 8 * PJ; sl < R; sl += 8) {
          float xv[4];
          Ring4<T>::ld(rb + (size_t)((t - sl) & (R - 1)) * d, xv);
          const float m = (t - sl >= 0) ? 1.f : 0.f;
#pragma unroll
          for (int v = 0; v < 4; ++v) xv[v] *= m;
          if constexpr (!prime) {
            const float4 rv = *(const float4*)(fir + (size_t)sl * d + c);
            f[0] = fmaf(rv.x, xv[0], f[0]);
            f[1] = fmaf(rv.y, xv[1], f[1]);
            f[2] = fmaf(rv.z, xv[2], f[2]);
            f[3] = fmaf(rv.w, xv[3], f[3]);
          }
          if (OM != 0 && sl + 1 < R) {
            const float4 rv2 = *(const float4*)(fir + (size_t)(sl + 1) * d + c);
            fnx[0] = fmaf(rv2.x, xv[0], fnx[0]);
            fnx[1] = fmaf(rv2.y, xv[1], fnx[1]);
            fnx[2] = fmaf(rv2.z, xv[2], fnx[2]);
            fnx[3] = fmaf(rv2.w, xv[3], fnx[3]);
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          if (jg & 1) acco[v] += f[v]; else acc[v] += f[v];
        }
      }
      if (head && jg == 0 && !prime) Ring4<T>::st(ring + ((size_t)b * R + (t & (R - 1))) * d + c, x);
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) { sh[jg][q][v] = acc[v]; sho[jg][q][v] = acco[v]; }
  if (omode && (jg & 1) == 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) shf[jg + 1][q][v] = fnx[v];
  }
  __syncthreads();
  if (jg == 0 && ok) {
    float onext[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float e = 0.f, o = 0.f;
#pragma unroll
      for (int g = 0; g < LDS_JG; ++g) {
        e += sh[g][q][v];
        // (omode: what the plain step's odd mode group g holds before the reduction: its bank sum plus its lags)
        o += (omode && head && (g & 1)) ? sho[g][q][v] + shf[g][q][v] : sho[g][q][v];
      }
      onext[v] = o;
      if (omode) o = ocur[v];
      if constexpr (!prime) {
        const float out = pair ? DT<T>::rnd(e + o) + DT<T>::rnd(e - o) : scale * (e + o);
        DT<T>::st(y + (size_t)b * ldy + c + v, res ? rsd[v] + DT<T>::rnd(out) : out);
      }
    }
    if (omode) Ring4<float>::st(ocache + (size_t)b * d + c, onext);
  }
}

extern "C" int fstu_stu_step_lds(float* state, const void* xp, int ldxp, const float* a, const float* ce, void* y,
                                 int ldy, int B, int S, int d, int t, int dtype, void* stream) {
  return fstu_stu_step_lds_dyn(state, xp, ldxp, a, ce, y, ldy, B, S, d, t, nullptr, dtype, stream);
}

static int stu_step_lds_launch(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                               float scale, void* y, int ldy, int B, int S, int d, int t, const int* dyn, int dtype,
                               void* stream, int pair = 0, void* ring = nullptr, const float* fir = nullptr, int R = 0,
                               const int* pos_dyn = nullptr, const void* res = nullptr, float* ocache = nullptr, int omode = 0);

int fstu_stu_step_lds_dyn(float* state, const void* xp, int ldxp, const float* a, const float* ce, void* y, int ldy,
                          int B, int S, int d, int t, const int* dyn, int dtype, void* stream) {
  return stu_step_lds_launch(state, xp, ldxp, a, ce, nullptr, 2.0f, y, ldy, B, S, d, t, dyn, dtype, stream);
}

extern "C" int fstu_stu_step_lds_single(float* state, const void* xp, int ldxp, const float* a, const float* ce,
                                        const float* co, void* y, int ldy, int B, int S, int d, int t, int dtype,
                                        void* stream) {
  FSTU_REQUIRE(co, FSTU_ENULL, "fstu_stu_step_lds_single: null pointer");
  FSTU_REQUIRE(fstu_aligned(co, 16), FSTU_EALIGN, "fstu_stu_step_lds_single: co must be 16-byte aligned");
  return stu_step_lds_launch(state, xp, ldxp, a, ce, co, 1.0f, y, ldy, B, S, d, t, nullptr, dtype, stream);
}

extern "C" int fstu_stu_step_lds_pair(float* state, const void* xp, int ldxp, const float* a, const float* ce,
                                      const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, int B, int S,
                                      int d, int t, int dtype, void* stream) {
  return fstu_stu_step_lds_pair_dyn(state, xp, ldxp, a, ce, co, ring, fir, fir_taps, y, ldy, B, S, d, t, nullptr, nullptr, dtype,
                                    stream, nullptr, nullptr);
}

// ring / fir / fir_taps: optional exact head of the filter (all three or none).  dyn: device-side {position, step} that
// supplies the parity; pos_dyn: the same words where only the ring slot is read from them (the parity then comes with t)
int fstu_stu_step_lds_pair_dyn(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co, void* ring,
                               const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int t, const int* dyn,
                               const int* pos_dyn, int dtype, void* stream, const void* res, float* ocache) {
  FSTU_REQUIRE(co, FSTU_ENULL, "fstu_stu_step_lds_pair: null pointer");
  FSTU_REQUIRE(fstu_aligned(co, 16), FSTU_EALIGN, "fstu_stu_step_lds_pair: co must be 16-byte aligned");
  FSTU_REQUIRE(fstu_fir_ok(ring, fir, fir_taps), FSTU_EARG,
               "fstu_stu_step_lds_pair: ring, fir and fir_taps (a power of two, 8..1024) go together, 16-byte aligned");
  return stu_step_lds_launch(state, xp, ldxp, a, ce, co, 1.0f, y, ldy, B, S, d, t, dyn, dtype, stream, 1, ring, fir, fir_taps,
                             dyn ? dyn : pos_dyn, res, ocache, ocache ? 1 : 0);
}

// The pair step with the odd-lag sum handed from step to step: ocache (B,d) fp32 holds the O of position t (from the
// step at t-1 or from fstu_stu_step_lds_prime) and receives the O of position t+1, so the bank of the other parity
// is not read.  Same values as fstu_stu_step_lds_pair, bit for bit.  res may be NULL; otherwise as in _pair_add.
extern "C" int fstu_stu_step_lds_pair_cached(float* state, const void* xp, int ldxp, const float* a, const float* ce,
                                             const float* co, void* ring, const float* fir, int fir_taps, float* ocache,
                                             const void* res, void* y, int ldy, int B, int S, int d, int t, int dtype,
                                             void* stream) {
  FSTU_REQUIRE(ocache, FSTU_ENULL, "fstu_stu_step_lds_pair_cached: ocache is null");
  return fstu_stu_step_lds_pair_dyn(state, xp, ldxp, a, ce, co, ring, fir, fir_taps, y, ldy, B, S, d, t, nullptr, nullptr, dtype,
                                    stream, res, ocache);
}

// ocache = the O of position t+1 as a pair step at position t would leave it, from the state and the ring as they
// stand after position t (a prompt's last position): nothing else is read or written.
extern "C" int fstu_stu_step_lds_prime(const float* state, const float* a, const float* co, const void* ring, const float* fir,
                                       int fir_taps, float* ocache, int B, int S, int d, int t, int dtype, void* stream) {
  FSTU_REQUIRE(state && a && co && ocache, FSTU_ENULL, "fstu_stu_step_lds_prime: null pointer");
  FSTU_REQUIRE(fstu_aligned(co, 16), FSTU_EALIGN, "fstu_stu_step_lds_prime: co must be 16-byte aligned");
  FSTU_REQUIRE(fstu_fir_ok(ring, fir, fir_taps), FSTU_EARG,
               "fstu_stu_step_lds_prime: ring, fir and fir_taps (a power of two, 8..1024) go together, 16-byte aligned");
  // (ce, xp and y are not touched in this mode; valid pointers stand in for them)
  return stu_step_lds_launch(const_cast<float*>(state), ocache, d, a, co, co, 1.0f, ocache, d, B, S, d, t, nullptr, dtype, stream, 1,
                             const_cast<void*>(ring), fir, fir_taps, nullptr, nullptr, ocache, 2);
}

// The same step joining the residual stream: y = T(res + T(step output)), rows of stride ldy in both; y may be res
// (every element is read and written by the same thread).
extern "C" int fstu_stu_step_lds_pair_add(float* state, const void* xp, int ldxp, const float* a, const float* ce,
                                          const float* co, void* ring, const float* fir, int fir_taps, const void* res, void* y,
                                          int ldy, int B, int S, int d, int t, int dtype, void* stream) {
  FSTU_REQUIRE(res, FSTU_ENULL, "fstu_stu_step_lds_pair_add: res is null");
  return fstu_stu_step_lds_pair_dyn(state, xp, ldxp, a, ce, co, ring, fir, fir_taps, y, ldy, B, S, d, t, nullptr, nullptr, dtype,
                                    stream, res, nullptr);
}

static int stu_step_lds_launch(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                               float scale, void* y, int ldy, int B, int S, int d, int t, const int* dyn, int dtype,
                               void* stream, int pair, void* ring, const float* fir, int R, const int* pos_dyn, const void* res,
                               float* ocache, int omode) {
  FSTU_REQUIRE(state && xp && a && ce && y, FSTU_ENULL, "fstu_stu_step_lds: null pointer");
  FSTU_REQUIRE(omode == 0 || (ocache && co && fstu_aligned(ocache, 16)), FSTU_EARG,
               "fstu_stu_step_lds: the handed-on odd-lag sum needs co and a 16-byte aligned ocache");
  FSTU_REQUIRE(!res || (fstu_aligned(res, 16) && ldy % 4 == 0), FSTU_EALIGN,
               "fstu_stu_step_lds: the residual rows must be 16-byte aligned with a stride that is a multiple of 4");
  FSTU_REQUIRE(B >= 1 && S >= 1 && d >= 4 && d % 4 == 0, FSTU_ESHAPE, "fstu_stu_step_lds: need d %% 4 == 0 (B=%d S=%d d=%d)", B, S, d);
  FSTU_REQUIRE(ldxp >= d && ldy >= d, FSTU_ESHAPE, "fstu_stu_step_lds: row stride smaller than d");
  FSTU_REQUIRE(t >= 0, FSTU_EARG, "fstu_stu_step_lds: t<0");
  FSTU_REQUIRE(fstu_aligned(state, 16) && fstu_aligned(ce, 16), FSTU_EALIGN, "fstu_stu_step_lds: state/ce must be 16-byte aligned");
  dim3 grid((d / 4 + 31) / 32, B);
#define STU_STEP_GO(OM)                                                                                               \
  hipLaunchKernelGGL((stu_step_lds_kernel<T, OM>), grid, dim3(256), 0, (hipStream_t)stream, state, (const T*)xp, ldxp, a, ce, \
                     co, scale, (T*)y, ldy, S, d, t & 1, dyn, pair, (T*)ring, fir, R, t, pos_dyn, (const T*)res, ocache)
  FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_step_lds", {
    if (omode == 1) STU_STEP_GO(1); else if (omode == 2) STU_STEP_GO(2); else STU_STEP_GO(0);
  });
#undef STU_STEP_GO
  FSTU_CHECK_LAUNCH("fstu_stu_step_lds");
  return FSTU_OK;
}

// ---------------------------------------------------------------- exact mode: filter-bank step on the recurrence state
// One token of use_approx=False (flash_stu/modules/stu.py:99-120) without re-running the convolution: the two parity
// banks of state hold h_j = sum_m a_j^m x[t' - 2m] of the raw inputs; with ce/co (S,K) fitted to the even / odd lags
// of every filter phi_k,
//   E_k = sum_j ce[j,k] h_j[bank of t],  O_k = sum_j co[j,k] h_j[other bank]   (lag 2m+1 reaches x[t-1-2m])
//   U+[b,k,c] = T(E_k + O_k),  U-[b,k,c] = T(E_k - O_k)
// Thread = one (batch, channel); the fitted weights sit in LDS; state traffic is coalesced along the channels.
#define BANK_MAXK 32
template <typename T>
__global__ void __launch_bounds__(256)
stu_bank_step_kernel(float* __restrict__ state, const T* __restrict__ x, int ldx, const float* __restrict__ a,
                     const float* __restrict__ ce, const float* __restrict__ co, T* __restrict__ up, T* __restrict__ um,
                     int S, int d, int K, int parity, const int* __restrict__ dyn) {
  extern __shared__ float bank_smem[];   // a (S), ce (S*K), co (S*K)
  float* sa = bank_smem;
  float* sce = sa + S;
  float* sco = sce + (size_t)S * K;
  if (dyn) parity = dyn[0] & 1;
  for (int i = threadIdx.x; i < S; i += 256) sa[i] = a[i];
  for (int i = threadIdx.x; i < S * K; i += 256) {
    sce[i] = ce[i];
    sco[i] = co ? co[i] : 0.f;
  }
  __syncthreads();
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= d) return;
  const float xv = DT<T>::ld(x + (size_t)b * ldx + c);
  float* sp = state + (((size_t)b * 2 + parity) * S) * d + c;
  const float* sq = state + (((size_t)b * 2 + (1 - parity)) * S) * d + c;
  float E[BANK_MAXK], O[BANK_MAXK];
#pragma unroll
  for (int k = 0; k < BANK_MAXK; ++k) E[k] = O[k] = 0.f;
  for (int j = 0; j < S; ++j) {
    const float hp = fmaf(sa[j], sp[(size_t)j * d], xv);
    sp[(size_t)j * d] = hp;
    const float hq = sq[(size_t)j * d];
    const float* cej = sce + (size_t)j * K;
    const float* coj = sco + (size_t)j * K;
#pragma unroll
    for (int k = 0; k < BANK_MAXK; ++k) {
      if (k < K) {
        E[k] = fmaf(cej[k], hp, E[k]);
        O[k] = fmaf(coj[k], hq, O[k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < BANK_MAXK; ++k) {
    if (k < K) {
      DT<T>::st(up + ((size_t)b * K + k) * d + c, E[k] + O[k]);
      if (um) DT<T>::st(um + ((size_t)b * K + k) * d + c, E[k] - O[k]);
    }
  }
}

extern "C" int fstu_stu_bank_step_lds(float* state, const void* x, int ldx, const float* a, const float* ce, const float* co,
                                      void* u_plus, void* u_minus, int B, int S, int d, int K, int t, int dtype,
                                      void* stream) {
  FSTU_REQUIRE(state && x && a && ce && u_plus, FSTU_ENULL, "fstu_stu_bank_step_lds: null pointer");
  FSTU_REQUIRE(B >= 1 && B <= 65535 && S >= 1 && d >= 1 && K >= 1 && K <= BANK_MAXK && ldx >= d && t >= 0, FSTU_ESHAPE,
               "fstu_stu_bank_step_lds: bad shape B=%d S=%d d=%d K=%d (K <= %d)", B, S, d, K, BANK_MAXK);
  const size_t shm = (size_t)(S + 2 * S * K) * sizeof(float);
  FSTU_REQUIRE(shm <= 60 * 1024, FSTU_ESHAPE, "fstu_stu_bank_step_lds: S*K too large for LDS");
  dim3 grid((d + 255) / 256, B);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_bank_step_lds",
                      hipLaunchKernelGGL(stu_bank_step_kernel<T>, grid, dim3(256), shm, (hipStream_t)stream, state, (const T*)x,
                                         ldx, a, ce, co, (T*)u_plus, (T*)u_minus, S, d, K, t & 1, (const int*)nullptr));
  FSTU_CHECK_LAUNCH("fstu_stu_bank_step_lds");
  return FSTU_OK;
}

// ---------------------------------------------------------------- input projection + LDS-form step, one launch
// Workgroup = one tile of 16 channels x INPROJ_RB batch rows: x_proj[b, c] = T(h[b,:] . Mt[c,:]) by MFMA (K split over
// the 4 waves, reduced in LDS), then the recurrence step of those channels and rows.  The three operand streams of the
// step are dealt to different waves so that every load of the kernel is in flight before the projection and the whole
// kernel costs one trip to memory: wave 0 advances the bank of the token's parity (even lags), wave 1 reads the other
// bank (odd lags), waves 2 and 3 the exact head (ring of the last inputs).  Lane (cq, jsub, bsub) of a wave owns 4
// channels (float4) of row bsub and modes (or lags) jsub, jsub+8, ... (the head: jsub + 8*(wave-2), +16, ...).
typedef __bf16 stu_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float stu_floatx4_t __attribute__((ext_vector_type(4)));
#define INPROJ_RB 2

template <int PK /* chunks of 8 channels per thread in the norm prologue: rows * K / 8 <= PK * 256 */>
__global__ void __launch_bounds__(256)
stu_inproj_step_kernel(const bf16_t* __restrict__ h, const bf16_t* __restrict__ Mt /*(d,K) = M_inputs^T*/,
                       float* __restrict__ state, const float* __restrict__ a, const float* __restrict__ ce,
                       bf16_t* __restrict__ y, const int* __restrict__ dyn, int parity /* pointers and the parity first:
                       these are the kernel-argument dwords the command processor preloads */, int ldh, int ldy,
                       bf16_t* __restrict__ xp_out /*optional (B,d)*/, int B, int S, int d, int K,
                       const bf16_t* __restrict__ x_res /*optional (B,K): normalise it instead of reading h*/,
                       const bf16_t* __restrict__ norm_w, float eps,
                       const float* __restrict__ slices /*optional, with x_res: up to 4 fp32 (B,K) slices added first*/,
                       int nslices, bf16_t* __restrict__ x_out /*receives x_res + T(sum of slices); not x_res itself*/,
                       const float* __restrict__ co /*optional (S,d): odd-lag weights on the other bank; then
                       y = T(T(E+O) + T(E-O)) instead of T(2E)*/,
                       bf16_t* __restrict__ ring /*optional (B,R,d), with fir (R,d) and co: exact head of the filter*/,
                       const float* __restrict__ fir, int R, int t, const int* __restrict__ pos_dyn) {
  __shared__ float red[4][64][4];
  __shared__ float xps[INPROJ_RB][16];          // [row][channel in tile], bf16-rounded values
  __shared__ float part[2][3][INPROJ_RB][16];   // [E | O][wave 0 or 1, wave 2, wave 3][row][channel]
  extern __shared__ __align__(16) unsigned char inproj_smem[];   // with x_res: h rows (INPROJ_RB x (K+8)) bf16
  if (dyn) parity = dyn[0] & 1;
  if (pos_dyn) t = pos_dyn[0];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  // A tile's 16 channels are half a 128-byte line of every state and output-weight row.  Workgroups go round the 8
  // XCDs, so consecutive tiles are dealt to one XCD (workgroups i, i+8, ...): both halves of a line then meet in the
  // same L2 and the line comes from HBM once instead of twice.
  int tile = blockIdx.x;
  if ((gridDim.x & 15) == 0) tile = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int c0 = tile * 16;
  const int b0 = blockIdx.y * INPROJ_RB, rows = min(INPROJ_RB, B - b0);
  // residual update + norm of this workgroup's rows in the prologue
  typedef NormPrologue<256, PK, 4> Pro;
  Pro pro;
  const bool merged = x_res != nullptr && slices != nullptr;
  // ---- projection: A operand = Mt rows (channels), B operand = h rows (batch)
  const int kw = K >> 2;                                    // k range of this wave
  const bf16_t* wp = Mt + (size_t)min(c0 + r, d - 1) * K + w * kw + g * 16;
  const bool xrow = r < rows;
  const bf16_t* hp = h + (size_t)(b0 + (xrow ? r : 0)) * ldh + w * kw + g * 16;   // re-pointed at LDS by the norm prologue
  // ---- the operands of this wave's part of the step go in flight before the projection: they do not depend on it,
  // and fetched afterwards they would cost a second dependent trip to memory
  constexpr int PJ = 8;
  const int cq = lane & 3, jsub = (lane >> 2) & 7, bsub = lane >> 5;
  const int c = c0 + cq * 4;
  const bool live = bsub < rows && c < d;
  const int b = b0 + (live ? bsub : 0), cc = live ? c : 0;
  const bool head = w >= 2;
  const int gl = jsub + 8 * (w - 2);   // head: first lag of this lane; the lags of a lane share its parity
  float4 pa[PJ], pb[PJ];
  float paj[PJ];
  // branch-free inside a role (out-of-range lanes, modes and lags re-read a valid element and ignore it): a conditional
  // load would reach its use through a copy, and the copy's wait would hold back every load issued after it
  if (!head) {
    const float* st = state + (((size_t)b * 2 + (parity ^ w)) * S) * d + cc;
    const float* cw = ((w == 0 || !co) ? ce : co) + cc;
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int j = min(jsub + 8 * k, S - 1);
      pa[k] = *(const float4*)(st + (size_t)j * d);
      pb[k] = *(const float4*)(cw + (size_t)j * d);
      paj[k] = a[j];
    }
  } else if (fir) {
    const bf16_t* rb = ring + (size_t)b * R * d + cc;
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int s = min(gl + 16 * k, R - 1);
      const uint2 q = *(const uint2*)(rb + (size_t)((t - s) & (R - 1)) * d);
      pa[k] = make_float4(__uint_as_float(q.x << 16), __uint_as_float(q.x & 0xffff0000u), __uint_as_float(q.y << 16),
                          __uint_as_float(q.y & 0xffff0000u));
      pb[k] = *(const float4*)(fir + (size_t)s * d + cc);
      paj[k] = 0.f;
    }
  }
  stu_floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
  // first batch of projection weights in flight before the optional norm prologue
  uint4 wa[4][2], xa[4][2];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (u < (kw >> 6)) {
      const uint4* p = (const uint4*)(wp + (size_t)u * 64);
      wa[u][0] = p[0];
      wa[u][1] = p[1];
    }
  }
  const int ldn = K + 8;
  // The prologue's loads go last: the compiler starts their arithmetic (and so their waits) right behind them, and
  // loads issued after that point would cost a second trip to memory.  The loads above return first anyway.
  __builtin_amdgcn_sched_barrier(0);
  if (merged) {
    const bf16_t* xr = x_res + (size_t)b0 * K;
    const float* sl = slices + (size_t)b0 * K;
    const int whole = B * (K >> 3);   // chunks of a whole slice
    pro.issue(xr, sl, nslices, norm_w, rows, K, whole);
    bf16_t* hs = (bf16_t*)inproj_smem;
    __shared__ float ss_part[Pro::NPART];
    pro.reduce(ss_part, blockIdx.x == 0 ? x_out + (size_t)b0 * K : nullptr, rows, K);
    __syncthreads();
    pro.scale(ss_part, hs, ldn, rows, K, eps);
    __syncthreads();
    hp = hs + (size_t)(xrow ? r : 0) * ldn + w * kw + g * 16;
  } else if (x_res) {
    // h = rmsnorm(x_res) * norm_w for this workgroup's rows into LDS
    bf16_t* hs = (bf16_t*)inproj_smem;
    const bf16_t* xr = x_res + (size_t)b0 * K;
    const int nchunk = K >> 3;
    for (int q = threadIdx.x; q < rows * nchunk; q += 256) {
      const int row = q / nchunk, c8 = (q - row * nchunk) << 3;
      *(uint4*)(hs + (size_t)row * ldn + c8) = *(const uint4*)(xr + (size_t)q * 8);
    }
    __syncthreads();
    for (int row = w; row < rows; row += 4) {
      bf16_t* hr = hs + (size_t)row * ldn;
      float ss = 0.f;
      for (int c8 = lane * 8; c8 < K; c8 += 512) {
        uint4 v = *(const uint4*)(hr + c8);
        unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo = __uint_as_float(vw[i] << 16), hi = __uint_as_float(vw[i] & 0xffff0000u);
          ss = fmaf(lo, lo, ss);
          ss = fmaf(hi, hi, ss);
        }
      }
      ss = wave_sum(ss);
      const float rstd = rsqrtf(ss / (float)K + eps);
      for (int c8 = lane * 8; c8 < K; c8 += 512) {
        uint4 v = *(const uint4*)(hr + c8);
        uint4 wv = *(const uint4*)(norm_w + c8);
        unsigned vw[4] = {v.x, v.y, v.z, v.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo = (__uint_as_float(vw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16);
          float hi = (__uint_as_float(vw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u);
          vw[i] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
        }
        *(uint4*)(hr + c8) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
      }
    }
    __syncthreads();
    hp = hs + (size_t)(xrow ? r : 0) * ldn + w * kw + g * 16;
  }
  for (int i0 = 0; i0 < (kw >> 6); i0 += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i0 + u < (kw >> 6)) {
        if (i0 > 0) {
          const uint4* p = (const uint4*)(wp + (size_t)(i0 + u) * 64);
          wa[u][0] = p[0];
          wa[u][1] = p[1];
        }
        if (xrow) {
          const uint4* q = (const uint4*)(hp + (size_t)(i0 + u) * 64);
          xa[u][0] = q[0];
          xa[u][1] = q[1];
        } else {
          xa[u][0] = make_uint4(0, 0, 0, 0);
          xa[u][1] = make_uint4(0, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i0 + u < (kw >> 6)) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(stu_bf16x8_t, wa[u][0]), __builtin_bit_cast(stu_bf16x8_t, xa[u][0]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(stu_bf16x8_t, wa[u][1]), __builtin_bit_cast(stu_bf16x8_t, xa[u][1]), acc, 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) red[w][lane][i] = acc[i];
  __syncthreads();
  if (w == 0 && xrow) {
    // D layout: lane holds channels 4*g+i of batch row r
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = DT<bf16_t>::rnd(((red[0][lane][i] + red[1][lane][i]) + red[2][lane][i]) + red[3][lane][i]);
      xps[r][4 * g + i] = v;
      if (xp_out && c0 + 4 * g + i < d) xp_out[(size_t)(b0 + r) * d + c0 + 4 * g + i] = f32_to_bf16(v);
    }
  }
  __syncthreads();
  // ---- this wave's part of the step
  const int bl = live ? bsub : 0;
  const float x0 = xps[bl][cq * 4], x1 = xps[bl][cq * 4 + 1], x2 = xps[bl][cq * 4 + 2], x3 = xps[bl][cq * 4 + 3];
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  if (w == 0) {
    // even lags: advance the bank of the token's parity
    float* st = state + (((size_t)b * 2 + parity) * S) * d + cc;
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int j = jsub + 8 * k;
      if (j < S && live) {
        float4 hv = pa[k];
        hv.x = fmaf(paj[k], hv.x, x0);
        hv.y = fmaf(paj[k], hv.y, x1);
        hv.z = fmaf(paj[k], hv.z, x2);
        hv.w = fmaf(paj[k], hv.w, x3);
        *(float4*)(st + (size_t)j * d) = hv;
        sum.x = fmaf(pb[k].x, hv.x, sum.x);
        sum.y = fmaf(pb[k].y, hv.y, sum.y);
        sum.z = fmaf(pb[k].z, hv.z, sum.z);
        sum.w = fmaf(pb[k].w, hv.w, sum.w);
      }
    }
    if (live) {
#pragma unroll 8
      for (int j = jsub + 8 * PJ; j < S; j += 8) {
        float4 hv = *(float4*)(st + (size_t)j * d);
        const float4 cj = *(const float4*)(ce + (size_t)j * d + c);
        const float aj = a[j];
        hv.x = fmaf(aj, hv.x, x0);
        hv.y = fmaf(aj, hv.y, x1);
        hv.z = fmaf(aj, hv.z, x2);
        hv.w = fmaf(aj, hv.w, x3);
        *(float4*)(st + (size_t)j * d) = hv;
        sum.x = fmaf(cj.x, hv.x, sum.x);
        sum.y = fmaf(cj.y, hv.y, sum.y);
        sum.z = fmaf(cj.z, hv.z, sum.z);
        sum.w = fmaf(cj.w, hv.w, sum.w);
      }
    }
  } else if (w == 1) {
    // odd lags: lag 2m+1 reaches position t-1-2m, which the bank of the other parity holds (read only)
    if (co && live) {
#pragma unroll
      for (int k = 0; k < PJ; ++k) {
        if (jsub + 8 * k < S) {
          sum.x = fmaf(pb[k].x, pa[k].x, sum.x);
          sum.y = fmaf(pb[k].y, pa[k].y, sum.y);
          sum.z = fmaf(pb[k].z, pa[k].z, sum.z);
          sum.w = fmaf(pb[k].w, pa[k].w, sum.w);
        }
      }
      const float* so = state + (((size_t)b * 2 + (parity ^ 1)) * S) * d + c;
#pragma unroll 8
      for (int j = jsub + 8 * PJ; j < S; j += 8) {
        const float4 hv = *(const float4*)(so + (size_t)j * d);
        const float4 oj = *(const float4*)(co + (size_t)j * d + c);
        sum.x = fmaf(oj.x, hv.x, sum.x);
        sum.y = fmaf(oj.y, hv.y, sum.y);
        sum.z = fmaf(oj.z, hv.z, sum.z);
        sum.w = fmaf(oj.w, hv.w, sum.w);
      }
    }
  } else if (fir && live) {
    // exact head: lags gl, gl+16, ... of the ring; a position before the sequence contributes nothing
#pragma unroll
    for (int k = 0; k < PJ; ++k) {
      const int s = gl + 16 * k;
      if (s < R) {
        const float m = (t - s >= 0) ? 1.f : 0.f;
        sum.x = fmaf(pb[k].x, s == 0 ? x0 : m * pa[k].x, sum.x);
        sum.y = fmaf(pb[k].y, s == 0 ? x1 : m * pa[k].y, sum.y);
        sum.z = fmaf(pb[k].z, s == 0 ? x2 : m * pa[k].z, sum.z);
        sum.w = fmaf(pb[k].w, s == 0 ? x3 : m * pa[k].w, sum.w);
      }
    }
    const bf16_t* rb = ring + (size_t)b * R * d + c;
#pragma unroll 4
    for (int s = gl + 16 * PJ; s < R; s += 16) {
      float xv[4];
      Ring4<bf16_t>::ld(rb + (size_t)((t - s) & (R - 1)) * d, xv);
      const float m = (t - s >= 0) ? 1.f : 0.f;
      const float4 rv = *(const float4*)(fir + (size_t)s * d + c);
      sum.x = fmaf(rv.x, m * xv[0], sum.x);
      sum.y = fmaf(rv.y, m * xv[1], sum.y);
      sum.z = fmaf(rv.z, m * xv[2], sum.z);
      sum.w = fmaf(rv.w, m * xv[3], sum.w);
    }
    if (gl == 0) {
      const float xv[4] = {x0, x1, x2, x3};
      Ring4<bf16_t>::st(ring + ((size_t)b * R + (t & (R - 1))) * d + c, xv);
    }
  }
  // reduce over the 8 mode groups of a wave (lanes differing in bits 2..4): two rotations inside the row of 16 lanes, one
  // swizzle across the two rows.  The head keeps even and odd lags apart (the rotation by 4 lanes joins them): its
  // lanes with jsub 0 end with the even lags' sum, those with jsub 1 with the odd lags'.
  auto grp_sum = [head](float v) {
    const float u = v + fstu_dpp<0x124>(v);   // row_ror:4
    v = head ? v : u;
    v += fstu_dpp<0x128>(v);   // row_ror:8
    return v + fstu_swz16(v);
  };
  sum.x = grp_sum(sum.x);
  sum.y = grp_sum(sum.y);
  sum.z = grp_sum(sum.z);
  sum.w = grp_sum(sum.w);
  if (bsub < INPROJ_RB && jsub < (head ? 2 : 1)) {
    const int eo = head ? jsub : w;          // 0: joins E, 1: joins O
    const int src = head ? w - 1 : 0;
    float* pp = &part[eo][src][bsub][cq * 4];
    pp[0] = sum.x; pp[1] = sum.y; pp[2] = sum.z; pp[3] = sum.w;
  }
  __syncthreads();
  if (w == 0 && jsub == 0 && live) {
    float o4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float e = (part[0][0][bsub][cq * 4 + i] + part[0][1][bsub][cq * 4 + i]) + part[0][2][bsub][cq * 4 + i];
      const float o = (part[1][0][bsub][cq * 4 + i] + part[1][1][bsub][cq * 4 + i]) + part[1][2][bsub][cq * 4 + i];
      o4[i] = co ? DT<bf16_t>::rnd(e + o) + DT<bf16_t>::rnd(e - o) : 2.f * e;
    }
    bf16_t* yp = y + (size_t)b * ldy + c;
    if ((ldy & 3) == 0) {
      *(uint2*)yp = make_uint2(pack2_bf16(o4[0], o4[1]), pack2_bf16(o4[2], o4[3]));
    } else {
      yp[0] = f32_to_bf16(o4[0]);
      yp[1] = f32_to_bf16(o4[1]);
      yp[2] = f32_to_bf16(o4[2]);
      yp[3] = f32_to_bf16(o4[3]);
    }
  }
}
struct FirArgs {
  void* ring;
  const float* fir;
  int taps;
  const int* pos_dyn;
};
static int inproj_step_launch(const void* h, int ldh, const void* x_res, const void* norm_w, float eps, const void* Mt,
                              float* state, const float* a, const float* ce, const float* co, void* y, int ldy, void* xp_out,
                              int B, int S, int d, int K, int t, const int* dyn, void* stream, FirArgs fa,
                              const float* slices = nullptr, int nslices = 0, void* x_out = nullptr);

int fstu_stu_inproj_step_dyn(const void* h, int ldh, const void* Mt, float* state, const float* a, const float* ce,
                             const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, void* xp_out, int B,
                             int S, int d, int K, int t, const int* dyn, const int* pos_dyn, void* stream) {
  return inproj_step_launch(h, ldh, nullptr, nullptr, 0.f, Mt, state, a, ce, co, y, ldy, xp_out, B, S, d, K, t, dyn, stream,
                            FirArgs{ring, fir, fir_taps, dyn ? dyn : pos_dyn});
}

// x' = x_in + T(sum of nslices <= 4 fp32 slices) goes to x_out, h = rmsnorm(x') * norm_w feeds the projection: the
// add+norm launch between the previous layer's down projection and this layer, folded into this kernel
int fstu_stu_res_inproj_step_dyn(const void* x_in, const float* slices, int nslices, void* x_out, const void* norm_w, float eps,
                                 const void* Mt, float* state, const float* a, const float* ce, const float* co, void* ring,
                                 const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int K, int t,
                                 const int* dyn, const int* pos_dyn, void* stream) {
  FSTU_REQUIRE(x_in && slices && x_out && norm_w, FSTU_ENULL, "fstu_stu_res_inproj_step: null pointer");
  FSTU_REQUIRE(nslices >= 1 && nslices <= 4, FSTU_EARG, "fstu_stu_res_inproj_step: nslices=%d outside 1..4", nslices);
  FSTU_REQUIRE(x_out != x_in, FSTU_EARG, "fstu_stu_res_inproj_step: x_out must not alias x_in");
  FSTU_REQUIRE((NormPrologue<256, 4, 4>::supported(INPROJ_RB, K)), FSTU_ESHAPE, "fstu_stu_res_inproj_step: K=%d not supported", K);
  FSTU_REQUIRE(fstu_aligned(slices, 16) && fstu_aligned(x_out, 16), FSTU_EALIGN, "fstu_stu_res_inproj_step: pointers must be 16-byte aligned");
  return inproj_step_launch(x_in, K, x_in, norm_w, eps, Mt, state, a, ce, co, y, ldy, nullptr, B, S, d, K, t, dyn, stream,
                            FirArgs{ring, fir, fir_taps, dyn ? dyn : pos_dyn}, slices, nslices, x_out);
}

static int inproj_step_launch(const void* h, int ldh, const void* x_res, const void* norm_w, float eps, const void* Mt,
                              float* state, const float* a, const float* ce, const float* co, void* y, int ldy, void* xp_out,
                              int B, int S, int d, int K, int t, const int* dyn, void* stream, FirArgs fa, const float* slices,
                              int nslices, void* x_out) {
  FSTU_REQUIRE(h && Mt && state && a && ce && y, FSTU_ENULL, "fstu_stu_inproj_step: null pointer");
  FSTU_REQUIRE(fstu_fir_ok(fa.ring, fa.fir, fa.taps) && (!fa.fir || co), FSTU_EARG,
               "fstu_stu_inproj_step: ring, fir and fir_taps (a power of two, 8..1024) go together with co, 16-byte aligned");
  FSTU_REQUIRE(B >= 1 && B <= FSTU_MAX_DECODE_ROWS && S >= 1 && d >= 4 && d % 4 == 0, FSTU_ESHAPE, "fstu_stu_inproj_step: B=%d S=%d d=%d", B, S, d);
  FSTU_REQUIRE(K % 256 == 0 && ldh >= K && ldh % 8 == 0 && ldy >= d, FSTU_ESHAPE, "fstu_stu_inproj_step: K=%d must be a multiple of 256 (ldh=%d)", K, ldh);
  FSTU_REQUIRE(fstu_aligned(h, 16) && fstu_aligned(Mt, 16) && fstu_aligned(state, 16) && fstu_aligned(ce, 16), FSTU_EALIGN, "fstu_stu_inproj_step: pointers must be 16-byte aligned");
  const size_t shm = x_res ? (size_t)INPROJ_RB * (K + 8) * 2 : 0;
  FSTU_REQUIRE(shm <= 56 * 1024, FSTU_ESHAPE, "fstu_stu_inproj_step: B*K too large for the norm prologue");
  FSTU_REQUIRE(fstu_aligned(x_res, 16) && fstu_aligned(norm_w, 16) && fstu_aligned(co, 16), FSTU_EALIGN, "fstu_stu_inproj_step: x_res/norm_w/co must be 16-byte aligned");
  const dim3 grid((d + 15) / 16, (B + INPROJ_RB - 1) / INPROJ_RB);
#define INPROJ_LAUNCH(PK)                                                                                                  \
  hipLaunchKernelGGL(stu_inproj_step_kernel<PK>, grid, dim3(256), shm, (hipStream_t)stream, (const bf16_t*)h,             \
                     (const bf16_t*)Mt, state, a, ce, (bf16_t*)y, dyn, t & 1, ldh, ldy, (bf16_t*)xp_out, B, S, d, K,       \
                     (const bf16_t*)x_res, (const bf16_t*)norm_w, eps, slices, nslices, (bf16_t*)x_out, co,                \
                     (bf16_t*)fa.ring, fa.fir, fa.taps, t, fa.pos_dyn)
  const int chunks = INPROJ_RB * (K >> 3);
  if (chunks <= 256) INPROJ_LAUNCH(1);
  else if (chunks <= 512) INPROJ_LAUNCH(2);
  else INPROJ_LAUNCH(4);
#undef INPROJ_LAUNCH
  FSTU_CHECK_LAUNCH("fstu_stu_inproj_step");
  return FSTU_OK;
}

extern "C" int fstu_stu_res_inproj_step(const void* x_in, const float* slices, int nslices, void* x_out, const void* norm_w,
                                        float eps, const void* Mt, float* state, const float* a, const float* ce,
                                        const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, int B,
                                        int S, int d, int K, int t, void* stream) {
  return fstu_stu_res_inproj_step_dyn(x_in, slices, nslices, x_out, norm_w, eps, Mt, state, a, ce, co, ring, fir, fir_taps, y, ldy,
                                      B, S, d, K, t, nullptr, nullptr, stream);
}

extern "C" int fstu_stu_inproj_step(const void* h, int ldh, const void* Mt, float* state, const float* a, const float* ce,
                                    const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, void* xp_out,
                                    int B, int S, int d, int K, int t, void* stream) {
  return fstu_stu_inproj_step_dyn(h, ldh, Mt, state, a, ce, co, ring, fir, fir_taps, y, ldy, xp_out, B, S, d, K, t, nullptr, nullptr,
                                  stream);
}

// ---------------------------------------------------------------- state from history
#define LSH_JG 4
#define LSH_MAXJ 32
// element t of a (batch, channel) column through a raw buffer load: beyond the descriptor's range the load returns
// zero without a branch, so a whole batch of loads sits in straight-line code and can stay in flight while the
// previous batch is consumed
template <typename T> __device__ __forceinline__ float lsh_load(__amdgpu_buffer_rsrc_t rs, unsigned off);
template <> __device__ __forceinline__ float lsh_load<float>(__amdgpu_buffer_rsrc_t rs, unsigned off) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, 0));
}
template <> __device__ __forceinline__ float lsh_load<bf16_t>(__amdgpu_buffer_rsrc_t rs, unsigned off) {
  return bf16_to_f32((bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, off, 0, 0));
}

template <typename T, int MAXJ, int NG /* waves of a workgroup, each with up to MAXJ modes of the same 64 channels */>
__global__ void __launch_bounds__(NG * 64)
lds_state_from_hist_kernel(const T* __restrict__ hist, const float* __restrict__ a, float* __restrict__ state, int S,
                           int d, int t_last, int cap, T* __restrict__ ring /*optional (B,R,d): the last R inputs*/, int R) {
  const int b = blockIdx.y, p = blockIdx.z;
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int jg = threadIdx.x >> 6;
  const int per = (S + NG - 1) / NG;
  const int j0 = jg * per;
  if (c >= d) return;
  float h[MAXJ], aj[MAXJ];
#pragma unroll
  for (int i = 0; i < MAXJ; ++i) {
    h[i] = 0.f;
    aj[i] = (i < per && j0 + i < S) ? a[j0 + i] : 0.f;
  }
  // one descriptor per batch row: (t_last+1) rows of d elements
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(hist + (size_t)b * cap * d), 0, (unsigned)((size_t)(t_last + 1) * d * sizeof(T)), 0x00020000);
  const unsigned row = (unsigned)d * (unsigned)sizeof(T), col = (unsigned)c * (unsigned)sizeof(T);
  // LSH_D batches of 16 positions are in flight: a batch is a quarter of a microsecond of arithmetic, a load a trip to
  // memory of one to two microseconds
  constexpr int LSH_D = 4;
  float xq[LSH_D][16];
#pragma unroll
  for (int u = 0; u < LSH_D; ++u)
#pragma unroll
    for (int k = 0; k < 16; ++k) xq[u][k] = lsh_load<T>(rs, (unsigned)(p + 32 * u + 2 * k) * row + col);
  for (int tt0 = p; tt0 <= t_last; tt0 += 32 * LSH_D) {
#pragma unroll
    for (int u = 0; u < LSH_D; ++u) {
      float xs[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) xs[k] = xq[u][k];
#pragma unroll
      for (int k = 0; k < 16; ++k) xq[u][k] = lsh_load<T>(rs, (unsigned)(tt0 + 32 * (LSH_D + u) + 2 * k) * row + col);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (tt0 + 32 * u + 2 * k <= t_last) {      // a step past the end must not decay the state
#pragma unroll
          for (int i = 0; i < MAXJ; ++i) h[i] = fmaf(aj[i], h[i], xs[k]);
        }
      }
      // the exact head's ring: position t in slot t % R for the last R positions, written by the first wave on the way
      // (every slot is covered when the sequence has R positions; a shorter one leaves the others as the caller zeroed them)
      if (ring && jg == 0 && tt0 + 32 * u + 30 > t_last - R) {
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          const int t = tt0 + 32 * u + 2 * k;
          if (t <= t_last && t > t_last - R) DT<T>::st(ring + ((size_t)b * R + (t & (R - 1))) * d + c, xs[k]);
        }
      }
    }
  }
  float* st = state + (((size_t)b * 2 + p) * S) * d + c;
#pragma unroll
  for (int i = 0; i < MAXJ; ++i)
    if (i < per && j0 + i < S) st[(size_t)(j0 + i) * d] = h[i];
}

extern "C" int fstu_stu_lds_state_from_hist(const void* hist, const float* a, float* state, int B, int S, int d,
                                            int t_last, int cap, int dtype, void* stream) {
  return fstu_stu_lds_state_ring_from_hist(hist, a, state, nullptr, 0, B, S, d, t_last, cap, dtype, stream);
}

extern "C" int fstu_stu_lds_state_ring_from_hist(const void* hist, const float* a, float* state, void* ring, int R, int B, int S,
                                                 int d, int t_last, int cap, int dtype, void* stream) {
  FSTU_REQUIRE(hist && a && state, FSTU_ENULL, "fstu_stu_lds_state_from_hist: null pointer");
  FSTU_REQUIRE(ring == nullptr || (R >= 8 && R <= 1024 && (R & (R - 1)) == 0), FSTU_EARG,
               "fstu_stu_lds_state_ring_from_hist: ring length %d is not a power of two in 8..1024", R);
  FSTU_REQUIRE(B >= 1 && d >= 1 && S >= 1 && S <= LSH_JG * LSH_MAXJ, FSTU_ESHAPE,
               "fstu_stu_lds_state_from_hist: S=%d outside 1..%d", S, LSH_JG * LSH_MAXJ);
  FSTU_REQUIRE(t_last >= -1 && t_last < cap, FSTU_EARG, "fstu_stu_lds_state_from_hist: t_last=%d cap=%d", t_last, cap);
  FSTU_REQUIRE((size_t)cap * d * 4 < 0xfff00000ull, FSTU_ESHAPE, "fstu_stu_lds_state_from_hist: cap*d too large for 32-bit offsets");
  dim3 grid((d + 63) / 64, B, 2);
  if (S <= 64) {
    // 8 waves of 8 modes: two waves per SIMD cover each other's dependent fused multiply-adds
    FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_lds_state_from_hist",
                        hipLaunchKernelGGL((lds_state_from_hist_kernel<T, 8, 8>), grid, dim3(512), 0, (hipStream_t)stream,
                                           (const T*)hist, a, state, S, d, t_last, cap, (T*)ring, R));
  } else {
    FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_lds_state_from_hist",
                        hipLaunchKernelGGL((lds_state_from_hist_kernel<T, LSH_MAXJ, LSH_JG>), grid, dim3(256), 0,
                                           (hipStream_t)stream, (const T*)hist, a, state, S, d, t_last, cap, (T*)ring, R));
  }
  FSTU_CHECK_LAUNCH("fstu_stu_lds_state_from_hist");
  return FSTU_OK;
}

// ---------------------------------------------------------------- whole-sequence recurrence (scan form of the prefill)
// The decode step of fstu_stu_step_lds applied to T consecutive positions in one launch: outputs for every position and
// the state after the last one, without an FFT and without a history buffer (sequence counterpart of
// mini_stu/stu_lds.py:17-68,279-338).  The two parity banks are independent recurrences (even positions only touch
// the even bank), so they advance side by side: workgroup = (32 channels, batch row), lane = (parity, channel), and
// one pass of the loop steps an even and an odd position.  The 8 waves split the modes; wave w keeps modes
// [w*MW, (w+1)*MW) of its lanes' bank in registers for the whole sequence.  Time runs in blocks of 32 positions: the
// block's inputs are staged in LDS once (the next block's are in flight meanwhile), every wave steps its modes
// through the block and leaves one partial output per position in LDS, then the 8 partials are summed in wave order.
// Per mode the update is the same fmaf as the decode step, so the final state equals T decode steps bit for bit;
// the outputs differ from them only by the order of the sum over modes.
#define SCAN_TB 32
#define SCAN_CH 32
template <typename T, int MW>
__global__ void __launch_bounds__(512)
stu_scan_lds_kernel(const T* __restrict__ xp, long long sxb, long long sxt, const float* __restrict__ a,
                    const float* __restrict__ ce, float* __restrict__ state, T* __restrict__ y, long long syb,
                    long long syt, int Tn, int S, int d, int t_start, int carry) {
  __shared__ __align__(16) T xs[SCAN_TB * SCAN_CH];
  __shared__ float part[8][SCAN_TB * SCAN_CH];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int ch = lane & 31, hp = lane >> 5;      // hp: parity of the position inside this call
  const int b = blockIdx.y, c0 = blockIdx.x * SCAN_CH, c = c0 + ch;
  const bool cok = c < d;
  const int cc = cok ? c : d - 1;
  const int bank = hp ^ (t_start & 1);           // the state bank this lane advances
  float h[MW], aj[MW], cj[MW];
#pragma unroll
  for (int m = 0; m < MW; ++m) {
    const int j = w * MW + m;
    const bool jok = j < S;
    aj[m] = jok ? a[j] : 0.f;
    cj[m] = jok ? ce[(size_t)j * d + cc] : 0.f;
    h[m] = (carry && jok) ? state[(((size_t)b * 2 + bank) * S + j) * d + cc] : 0.f;
  }
  // input tile: SCAN_TB rows of SCAN_CH channels, one 16-byte piece per loading thread
  constexpr int PIECES = SCAN_TB * SCAN_CH * (int)sizeof(T) / 16, PPR = SCAN_CH * (int)sizeof(T) / 16,
                EPP = 16 / (int)sizeof(T);
  const int prow = threadIdx.x / PPR, pcol = (threadIdx.x % PPR) * EPP;
  const bool ploader = threadIdx.x < PIECES && c0 + pcol < d;
  auto load_tile = [&](int t0) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (ploader && t0 + prow < Tn) v = *(const uint4*)(xp + (size_t)b * sxb + (size_t)(t0 + prow) * sxt + c0 + pcol);
    return v;
  };
  uint4 xr = load_tile(0);
  for (int t0 = 0; t0 < Tn; t0 += SCAN_TB) {
    if (threadIdx.x < PIECES) *(uint4*)(xs + prow * SCAN_CH + pcol) = xr;
    __syncthreads();
    xr = load_tile(t0 + SCAN_TB);
#pragma unroll
    for (int i = 0; i < SCAN_TB / 2; ++i) {
      // position 2i + hp of the block: element 64 i + lane of the tile
      float p = 0.f;
      if (t0 + 2 * i + hp < Tn) {   // a step past the end must not decay the state
        const float x = DT<T>::ld(xs + 64 * i + lane);
#pragma unroll
        for (int m = 0; m < MW; ++m) {
          h[m] = fmaf(aj[m], h[m], x);
          p = fmaf(cj[m], h[m], p);
        }
      }
      part[w][64 * i + lane] = p;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < SCAN_TB / 16; ++i) {
      const int e = (w * (SCAN_TB / 16) + i) * 64 + lane, k = e >> 5;   // tile element: position k, channel ch
      float sum = 0.f;
#pragma unroll
      for (int ww = 0; ww < 8; ++ww) sum += part[ww][e];
      if (cok && t0 + k < Tn) DT<T>::st(y + (size_t)b * syb + (size_t)(t0 + k) * syt + c, 2.f * sum);
    }
  }
  if (cok) {
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const int j = w * MW + m;
      if (j < S) state[(((size_t)b * 2 + bank) * S + j) * d + c] = h[m];
    }
  }
}

extern "C" int fstu_stu_scan_lds(const void* xp, int64_t x_bstride, int64_t x_tstride, const float* a, const float* ce,
                                 float* state, void* y, int64_t y_bstride, int64_t y_tstride, int B, int len, int S, int d,
                                 int t_start, int carry, int dtype, void* stream) {
  FSTU_REQUIRE(xp && a && ce && state && y, FSTU_ENULL, "fstu_stu_scan_lds: null pointer");
  FSTU_REQUIRE(B >= 1 && B <= 65535 && len >= 0 && d >= 1 && S >= 1 && S <= 128 && t_start >= 0, FSTU_ESHAPE,
               "fstu_stu_scan_lds: B=%d T=%d S=%d d=%d t_start=%d (S <= 128)", B, len, S, d, t_start);
  const int epp = dtype == FSTU_BF16 ? 8 : 4;
  FSTU_REQUIRE(d % epp == 0 && x_tstride % epp == 0 && x_bstride % epp == 0 && fstu_aligned(xp, 16), FSTU_EALIGN,
               "fstu_stu_scan_lds: input rows must be 16-byte aligned (d and strides multiples of %d elements)", epp);
  FSTU_REQUIRE(x_tstride >= d && y_tstride >= d, FSTU_EARG, "fstu_stu_scan_lds: token stride below d");
  if (len == 0 && carry) return FSTU_OK;
  dim3 grid((d + SCAN_CH - 1) / SCAN_CH, B);
  hipStream_t s = (hipStream_t)stream;
  if (S <= 64) {
    FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_scan_lds",
                        hipLaunchKernelGGL((stu_scan_lds_kernel<T, 8>), grid, dim3(512), 0, s, (const T*)xp, (long long)x_bstride, (long long)x_tstride,
                                           a, ce, state, (T*)y, (long long)y_bstride, (long long)y_tstride, len, S, d, t_start, carry));
  } else {
    FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_scan_lds",
                        hipLaunchKernelGGL((stu_scan_lds_kernel<T, 16>), grid, dim3(512), 0, s, (const T*)xp, (long long)x_bstride, (long long)x_tstride,
                                           a, ce, state, (T*)y, (long long)y_bstride, (long long)y_tstride, len, S, d, t_start, carry));
  }
  FSTU_CHECK_LAUNCH("fstu_stu_scan_lds");
  return FSTU_OK;
}

// ---------------------------------------------------------------- direct prefill convolution
// Thread = (channel, tile of 16 output positions).  The 16 filter taps that
// meet the current input row form a sliding window in registers: advancing the
// input row by one shifts the window by one tap.
// The filter element of (lag, channel c) is filt[lag*f_ls + c*f_cs], so the same
// kernel serves a per-channel filter (f_ls=d, f_cs=1) and one column of a
// shared filter bank (f_ls=K, f_cs=0).  Output rows are ldy elements apart.
// mode 0: y = T(E+O) + T(E-O);  mode 1: y = T(E+O);  mode 2: y = T(E+O), y2 = T(E-O).
#define CONV_TT 16
template <typename T>
__global__ void __launch_bounds__(256)
stu_conv_direct_kernel(const T* __restrict__ xp, const T* __restrict__ filt, size_t f_ls, size_t f_cs,
                       T* __restrict__ y, T* __restrict__ y2, size_t ldy, int Tn, int d, int L, int mode) {
  const int b = blockIdx.z;
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int t0 = (blockIdx.y * 4 + (threadIdx.x >> 6)) * CONV_TT;
  if (c >= d || t0 >= Tn) return;
  const T* fc = filt + (size_t)c * f_cs;
  float aE[CONV_TT], aO[CONV_TT], fw[CONV_TT];
#pragma unroll
  for (int i = 0; i < CONV_TT; ++i) {
    aE[i] = 0.f;
    aO[i] = 0.f;
    int lag = t0 + i;
    fw[i] = (lag < L) ? DT<T>::ld(fc + (size_t)lag * f_ls) : 0.f;
  }
  const T* xb = xp + (size_t)b * Tn * d + c;
  const int ulast = min(Tn - 1, t0 + CONV_TT - 1);
  for (int u = 0; u <= ulast; ++u) {
    const float xv = DT<T>::ld(xb + (size_t)u * d);
    const int sel = (t0 - u) & 1;  // parity of the lag seen by output i=0
    if (sel == 0) {
#pragma unroll
      for (int i = 0; i < CONV_TT; ++i) {
        if (i & 1) aO[i] = fmaf(fw[i], xv, aO[i]); else aE[i] = fmaf(fw[i], xv, aE[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < CONV_TT; ++i) {
        if (i & 1) aE[i] = fmaf(fw[i], xv, aE[i]); else aO[i] = fmaf(fw[i], xv, aO[i]);
      }
    }
#pragma unroll
    for (int i = CONV_TT - 1; i > 0; --i) fw[i] = fw[i - 1];
    const int lag = t0 - u - 1;
    fw[0] = (lag >= 0 && lag < L) ? DT<T>::ld(fc + (size_t)lag * f_ls) : 0.f;
  }
  T* yb = y + (size_t)b * Tn * ldy + c;
  T* yb2 = (mode == 2) ? y2 + (size_t)b * Tn * ldy + c : nullptr;
#pragma unroll
  for (int i = 0; i < CONV_TT; ++i) {
    int t = t0 + i;
    if (t < Tn) {
      if (mode == 0) {
        DT<T>::st(yb + (size_t)t * ldy, DT<T>::rnd(aE[i] + aO[i]) + DT<T>::rnd(aE[i] - aO[i]));
      } else {
        DT<T>::st(yb + (size_t)t * ldy, aE[i] + aO[i]);
        if (mode == 2) DT<T>::st(yb2 + (size_t)t * ldy, aE[i] - aO[i]);
      }
    }
  }
}

extern "C" int fstu_stu_conv_direct(const void* xp, const void* filt, void* y, int B, int T_, int d, int L,
                                    int single_branch, int dtype, void* stream) {
  FSTU_REQUIRE(xp && filt && y, FSTU_ENULL, "fstu_stu_conv_direct: null pointer");
  FSTU_REQUIRE(B >= 1 && T_ >= 1 && d >= 1 && L >= 1 && B <= 65535, FSTU_ESHAPE, "fstu_stu_conv_direct: bad shape B=%d T=%d d=%d L=%d", B, T_, d, L);
  dim3 grid((d + 63) / 64, (T_ + 4 * CONV_TT - 1) / (4 * CONV_TT), B);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_conv_direct",
                      hipLaunchKernelGGL(stu_conv_direct_kernel<T>, grid, dim3(256), 0, (hipStream_t)stream,
                                         (const T*)xp, (const T*)filt, (size_t)d, (size_t)1, (T*)y, (T*)nullptr,
                                         (size_t)d, T_, d, L, single_branch ? 1 : 0));
  FSTU_CHECK_LAUNCH("fstu_stu_conv_direct");
  return FSTU_OK;
}

extern "C" int fstu_stu_conv_bank(const void* x, const void* phi, void* u_plus, void* u_minus, int B, int T_, int d,
                                  int L, int K, int dtype, void* stream) {
  FSTU_REQUIRE(x && phi && u_plus, FSTU_ENULL, "fstu_stu_conv_bank: null pointer");
  FSTU_REQUIRE(B >= 1 && T_ >= 1 && d >= 1 && L >= 1 && K >= 1 && B <= 65535, FSTU_ESHAPE, "fstu_stu_conv_bank: bad shape B=%d T=%d d=%d L=%d K=%d", B, T_, d, L, K);
  dim3 grid((d + 63) / 64, (T_ + 4 * CONV_TT - 1) / (4 * CONV_TT), B);
  for (int k = 0; k < K; ++k) {
    FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_conv_bank",
                        hipLaunchKernelGGL(stu_conv_direct_kernel<T>, grid, dim3(256), 0, (hipStream_t)stream,
                                           (const T*)x, (const T*)phi + k, (size_t)K, (size_t)0,
                                           (T*)u_plus + (size_t)k * d, u_minus ? (T*)u_minus + (size_t)k * d : (T*)nullptr,
                                           (size_t)K * d, T_, d, L, u_minus ? 2 : 1));
  }
  FSTU_CHECK_LAUNCH("fstu_stu_conv_bank");
  return FSTU_OK;
}

// ---------------------------------------------------------------- dense LDS steps
// One workgroup per batch row; the state element s lives in a register of
// thread s for the whole launch.
template <typename T>
__global__ void __launch_bounds__(256)
lds_steps_kernel(float* __restrict__ h, const T* __restrict__ x, const float* __restrict__ A, const T* __restrict__ Bm,
                 const T* __restrict__ Cm, T* __restrict__ y, int Tn, int Bt, int d_in, int S, int d_out) {
  extern __shared__ float smem[];
  float* xs = smem;          // d_in
  float* hs = smem + d_in;   // S
  const int b = blockIdx.x, tid = threadIdx.x;
  float hreg = (tid < S) ? h[(size_t)b * S + tid] : 0.f;
  const float areg = (tid < S) ? A[tid] : 0.f;
  for (int t = 0; t < Tn; ++t) {
    const T* xt = x + ((size_t)t * Bt + b) * d_in;
    for (int k = tid; k < d_in; k += 256) xs[k] = DT<T>::ld(xt + k);
    __syncthreads();
    if (tid < S) {
      float u = 0.f;
      for (int k = 0; k < d_in; ++k) u = fmaf(xs[k], DT<T>::ld(Bm + (size_t)k * S + tid), u);
      hreg = hreg * areg + u;
      hs[tid] = hreg;
    }
    __syncthreads();
    T* yt = y + ((size_t)t * Bt + b) * d_out;
    for (int o = tid; o < d_out; o += 256) {
      float acc = 0.f;
      for (int s = 0; s < S; ++s) acc = fmaf(hs[s], DT<T>::ld(Cm + (size_t)s * d_out + o), acc);
      DT<T>::st(yt + o, acc);
    }
    __syncthreads();
  }
  if (tid < S) h[(size_t)b * S + tid] = hreg;
}

extern "C" int fstu_lds_steps(float* h, const void* x, const float* A, const void* Bm, const void* Cm, void* y,
                              int T_steps, int Bt, int d_in, int S, int d_out, int dtype, void* stream) {
  FSTU_REQUIRE(h && x && A && Bm && Cm && y, FSTU_ENULL, "fstu_lds_steps: null pointer");
  FSTU_REQUIRE(T_steps >= 0 && Bt >= 1 && d_in >= 1 && d_out >= 1, FSTU_ESHAPE, "fstu_lds_steps: bad shape");
  FSTU_REQUIRE(S >= 1 && S <= 256, FSTU_ESHAPE, "fstu_lds_steps: S=%d outside 1..256", S);
  FSTU_REQUIRE((size_t)(d_in + S) * 4 <= 64 * 1024, FSTU_ESHAPE, "fstu_lds_steps: d_in=%d too large for LDS staging", d_in);
  if (T_steps == 0) return FSTU_OK;
  size_t shm = (size_t)(d_in + S) * sizeof(float);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_lds_steps",
                      hipLaunchKernelGGL(lds_steps_kernel<T>, dim3(Bt), dim3(256), shm, (hipStream_t)stream, h,
                                         (const T*)x, A, (const T*)Bm, (const T*)Cm, (T*)y, T_steps, Bt, d_in, S, d_out));
  FSTU_CHECK_LAUNCH("fstu_lds_steps");
  return FSTU_OK;
}
