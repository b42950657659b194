// Sliding-window attention with ALiBi and tanh soft-capping: ring KV cache
// maintenance, the single-query decode kernel and a simple prefill kernel.
//
// Work split: 8 lanes share one key (each lane owns hd/8 head dims), so a wave
// visits 8 keys at a time and a lane reads 16..64 contiguous bytes per key.
// Each 8-lane group keeps an online-softmax partial (max, sum, weighted V);
// partials are merged through LDS at the end.
#include "fstu_common.h"
#include "fstu_prologue.h"

template <typename T, int N>
__device__ __forceinline__ void load_vec(const T* p, float* o);

template <> __device__ __forceinline__ void load_vec<bf16_t, 4>(const bf16_t* p, float* o) {
  uint2 v = *(const uint2*)p;
  o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
  o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}
template <> __device__ __forceinline__ void load_vec<bf16_t, 8>(const bf16_t* p, float* o) {
  uint4 v = *(const uint4*)p;
  unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
}
template <> __device__ __forceinline__ void load_vec<bf16_t, 16>(const bf16_t* p, float* o) {
  load_vec<bf16_t, 8>(p, o);
  load_vec<bf16_t, 8>(p + 8, o + 8);
}
template <> __device__ __forceinline__ void load_vec<bf16_t, 32>(const bf16_t* p, float* o) {
  load_vec<bf16_t, 16>(p, o);
  load_vec<bf16_t, 16>(p + 16, o + 16);
}
// the same for data read exactly once per launch (the rings of a decode step): non-temporal, so that the stream does
// not push the step's weights and activations out of the caches
typedef unsigned swa_u32x4_t __attribute__((ext_vector_type(4)));
template <typename T, int N>
__device__ __forceinline__ void load_vec_stream(const T* p, float* o) { load_vec<T, N>(p, o); }
template <> __device__ __forceinline__ void load_vec_stream<bf16_t, 8>(const bf16_t* p, float* o) {
  const swa_u32x4_t v = __builtin_nontemporal_load((const swa_u32x4_t*)p);
#pragma unroll
  for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(v[i] << 16); o[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u); }
}
template <> __device__ __forceinline__ void load_vec_stream<bf16_t, 16>(const bf16_t* p, float* o) {
  load_vec_stream<bf16_t, 8>(p, o);
  load_vec_stream<bf16_t, 8>(p + 8, o + 8);
}
template <> __device__ __forceinline__ void load_vec_stream<bf16_t, 32>(const bf16_t* p, float* o) {
  load_vec_stream<bf16_t, 16>(p, o);
  load_vec_stream<bf16_t, 16>(p + 16, o + 16);
}
template <> __device__ __forceinline__ void load_vec<float, 4>(const float* p, float* o) {
  float4 v = *(const float4*)p;
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
template <> __device__ __forceinline__ void load_vec<float, 8>(const float* p, float* o) {
  load_vec<float, 4>(p, o); load_vec<float, 4>(p + 4, o + 4);
}
template <> __device__ __forceinline__ void load_vec<float, 16>(const float* p, float* o) {
  load_vec<float, 8>(p, o); load_vec<float, 8>(p + 8, o + 8);
}
template <> __device__ __forceinline__ void load_vec<float, 32>(const float* p, float* o) {
  load_vec<float, 16>(p, o); load_vec<float, 16>(p + 16, o + 16);
}

// A head-dim vector dealt to the 8 lanes of a key group in 16-byte pieces: piece p of lane gl holds elements
// p*8*E + gl*E .. +E (E = elements per 16 bytes), so every load instruction of the group covers 128 contiguous bytes of
// the row.  (With DPL consecutive elements per lane a 256-byte row was touched in every other 16 bytes by each of the
// two instructions: every line fetched twice.)
template <typename T, int DPL, bool STREAM>
__device__ __forceinline__ void load_pieces(const T* vec, int gl, float* o) {
  constexpr int E = 16 / (int)sizeof(T);
  if constexpr (DPL < E) {          // a row of less than 128 bytes: one short piece per lane
    load_vec<T, DPL>(vec + gl * DPL, o);
  } else {
#pragma unroll
    for (int p = 0; p < DPL / E; ++p) {
      if constexpr (STREAM) load_vec_stream<T, E>(vec + p * 8 * E + gl * E, o + p * E);
      else load_vec<T, E>(vec + p * 8 * E + gl * E, o + p * E);
    }
  }
}
template <typename T, int DPL>
__device__ __forceinline__ int piece_elem(int gl, int i) {   // element of the head-dim vector held in slot i of lane gl
  constexpr int E = 16 / (int)sizeof(T);
  if constexpr (DPL < E) return gl * DPL + i;
  return (i / E) * 8 * E + gl * E + (i % E);
}

// Online-softmax partial of one 8-lane key group.
template <int DPL>
struct Partial {
  float m, l;
  float acc[DPL];
};

// sum over each aligned group of 8 lanes, returned in every lane of the group (DPP, no LDS traffic)
template <int CTRL>
__device__ __forceinline__ float swa_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float group8_sum(float v) {
  v += swa_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  v += swa_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  v += swa_dpp<0x141>(v);   // row_half_mirror: the other quad of the 8
  return v;
}

// softcap * tanh(s / softcap).  FAST (bf16 models): tanh(t) = 1 - 2 / (exp(2t) + 1) on the hardware exp2 and
// reciprocal, absolute error about 1e-7 * softcap, far below the bf16 rounding of the operands; the fp32 parity
// path keeps tanhf.
template <bool FAST>
__device__ __forceinline__ float soft_cap(float s, float softcap, float inv_cap2l) {
  if (FAST) {
    const float e = __builtin_amdgcn_exp2f(s * inv_cap2l);   // exp(2 s / softcap)
    return softcap - (2.0f * softcap) * __builtin_amdgcn_rcpf(e + 1.0f);
  }
  return softcap * tanhf(s / softcap);
}

// One key for an 8-lane group: score, soft-cap, ALiBi, online-softmax update.  All 8 lanes of the group call it.
template <int DPL, bool FAST>
__device__ __forceinline__ void attend_one(Partial<DPL>& P, const float* q, const float* kk, const float* vv, int j, int pos,
                                           float scale, float softcap, float slope) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < DPL; ++i) s = fmaf(q[i], kk[i], s);
  s = group8_sum(s);
  s *= scale;
  if (softcap > 0.f) s = soft_cap<FAST>(s, softcap, 2.8853900817779268f / softcap);
  s -= slope * (float)(pos - j);
  float mn = fmaxf(P.m, s);
  float corr = __expf(P.m - mn);
  float p = __expf(s - mn);
  P.l = P.l * corr + p;
#pragma unroll
  for (int i = 0; i < DPL; ++i) P.acc[i] = fmaf(p, vv[i], P.acc[i] * corr);
  P.m = mn;
}

// Visits keys j = jb+u (u<U) for jb = j_first, j_first+j_step, ... < j_end.
// kb/vb point at this lane's dims of slot 0; consecutive slots are `stride`
// elements apart.  cap > 0: a ring, key j_lo sits in slot slot_lo (= j_lo % cap, computed once by the caller) and
// key j in slot_lo + (j - j_lo), wrapped once (j - j_lo < cap).  cap == 0: key j sits in slot j.
template <typename T, int DPL, int U, bool FAST>
__device__ __forceinline__ void attend_keys(Partial<DPL>& P, const T* kb, const T* vb, size_t stride, int cap, int j_lo,
                                            int slot_lo, const float* q, int j_first, int j_end, int j_step, int pos,
                                            float scale, float softcap, float slope) {
  const float inv_cap2l = softcap > 0.f ? 2.8853900817779268f / softcap : 0.f;
  for (int jb = j_first; jb < j_end; jb += j_step) {
    float kk[U][DPL], vv[U][DPL];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int j = jb + u;
      if (j < j_end) {
        int slot = j;
        if (cap > 0) {
          slot = slot_lo + (j - j_lo);
          slot = slot >= cap ? slot - cap : slot;
        }
        load_vec<T, DPL>(kb + (size_t)slot * stride, kk[u]);
        load_vec<T, DPL>(vb + (size_t)slot * stride, vv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int j = jb + u;
      const bool valid = j < j_end;  // uniform within the 8-lane group
      float s = 0.f;
      if (valid) {
#pragma unroll
        for (int i = 0; i < DPL; ++i) s = fmaf(q[i], kk[u][i], s);
      }
      s = group8_sum(s);
      if (valid) {
        s *= scale;
        if (softcap > 0.f) s = soft_cap<FAST>(s, softcap, inv_cap2l);
        s -= slope * (float)(pos - j);
        float mn = fmaxf(P.m, s);
        float corr = __expf(P.m - mn);
        float p = __expf(s - mn);
        P.l = P.l * corr + p;
#pragma unroll
        for (int i = 0; i < DPL; ++i) P.acc[i] = fmaf(p, vv[u][i], P.acc[i] * corr);
        P.m = mn;
      }
    }
  }
}

// ---------------------------------------------------------------- ring maintenance
template <typename T>
__global__ void kv_fill_kernel(const T* __restrict__ qkv, T* __restrict__ kring, T* __restrict__ vring, int B, int Tn,
                               int H, int hd, int cap, int pos0, int tstart) {
  // one thread per (b, tt, h, i) over tt in [tstart, Tn)
  const int d = H * hd;
  size_t n = (size_t)B * (Tn - tstart) * d;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
    int i = idx % hd;
    size_t r = idx / hd;
    int h = r % H;
    r /= H;
    int tt = tstart + (int)(r % (Tn - tstart));
    int b = (int)(r / (Tn - tstart));
    const T* src = qkv + ((size_t)b * Tn + tt) * 3 * d + h * hd + i;
    int slot = (pos0 + tt) % cap;
    size_t dst = (((size_t)b * H + h) * cap + slot) * hd + i;
    kring[dst] = src[d];
    vring[dst] = src[2 * d];
  }
}

// the same copy in 16-byte pieces (head dim a multiple of the piece, aligned pointers): one thread per piece
template <typename T>
__global__ void __launch_bounds__(256)
kv_fill_vec_kernel(const T* __restrict__ qkv, T* __restrict__ kring, T* __restrict__ vring, int B, int Tn, int H, int hd,
                   int cap, int pos0, int tstart) {
  constexpr int EPP = 16 / (int)sizeof(T);
  const int ppr = hd / EPP, d = H * hd, nt = Tn - tstart;
  const unsigned n = (unsigned)B * nt * H * ppr;
  for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < n; idx += gridDim.x * 256u) {
    const unsigned pc = idx % ppr, r1 = idx / ppr, h = r1 % H, r2 = r1 / H;
    const int tt = tstart + (int)(r2 % nt), b = (int)(r2 / nt);
    const T* src = qkv + ((size_t)b * Tn + tt) * 3 * d + h * hd + pc * EPP;
    const int slot = (pos0 + tt) % cap;
    const size_t dst = (((size_t)b * H + h) * cap + slot) * hd + pc * EPP;
    *(uint4*)(kring + dst) = *(const uint4*)(src + d);
    *(uint4*)(vring + dst) = *(const uint4*)(src + 2 * d);
  }
}

static int check_kv(const char* name, const void* a, const void* b, const void* c, int B, int H, int hd, int cap) {
  FSTU_REQUIRE(a && b && c, FSTU_ENULL, "%s: null pointer", name);
  FSTU_REQUIRE(B >= 1 && H >= 1 && hd >= 1 && cap >= 1, FSTU_ESHAPE, "%s: bad shape B=%d H=%d hd=%d cap=%d", name, B, H, hd, cap);
  return FSTU_OK;
}

extern "C" int fstu_kv_fill(const void* qkv, void* kring, void* vring, int B, int T_, int H, int hd, int cap, int pos0,
                            int dtype, void* stream) {
  int rc = check_kv("fstu_kv_fill", qkv, kring, vring, B, H, hd, cap);
  if (rc) return rc;
  FSTU_REQUIRE(T_ >= 1 && pos0 >= 0, FSTU_EARG, "fstu_kv_fill: T=%d pos0=%d", T_, pos0);
  int tstart = T_ > cap ? T_ - cap : 0;
  size_t n = (size_t)B * (T_ - tstart) * H * hd;
  unsigned blocks = (unsigned)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  const int epp = dtype == FSTU_BF16 ? 8 : 4;
  if (hd % epp == 0 && n / epp < 0xffffffffull && fstu_aligned(qkv, 16) && fstu_aligned(kring, 16) && fstu_aligned(vring, 16)) {
    const size_t np = n / epp;
    const unsigned vb = (unsigned)((np + 255) / 256 > 65535 ? 65535 : (np + 255) / 256);
    FSTU_DISPATCH_DTYPE(dtype, "fstu_kv_fill",
                        hipLaunchKernelGGL(kv_fill_vec_kernel<T>, dim3(vb), dim3(256), 0, (hipStream_t)stream,
                                           (const T*)qkv, (T*)kring, (T*)vring, B, T_, H, hd, cap, pos0, tstart));
    FSTU_CHECK_LAUNCH("fstu_kv_fill");
    return FSTU_OK;
  }
  FSTU_DISPATCH_DTYPE(dtype, "fstu_kv_fill",
                      hipLaunchKernelGGL(kv_fill_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                                         (const T*)qkv, (T*)kring, (T*)vring, B, T_, H, hd, cap, pos0, tstart));
  FSTU_CHECK_LAUNCH("fstu_kv_fill");
  return FSTU_OK;
}

extern "C" int fstu_kv_append(const void* qkv, void* kring, void* vring, int B, int H, int hd, int cap, int pos,
                              int dtype, void* stream) {
  FSTU_REQUIRE(pos >= 0, FSTU_EARG, "fstu_kv_append: pos<0");
  return fstu_kv_fill(qkv, kring, vring, B, 1, H, hd, cap, pos, dtype, stream);
}

// ---------------------------------------------------------------- decode
// One workgroup per (batch, head); NWAVES*8 key groups visit 4 keys each per
// sweep, so a 513-key window is covered in two sweeps with every load of a
// sweep in flight at once.  With append != 0 the workgroup stores the new token's
// k,v (read from the qkv row) into ring slot pos % cap and attends to that key
// straight from the qkv row, so the ring sweep covers the older keys only.
// STREAM: the ring loads are non-temporal.  The rings of a step that fit the memory-side cache next to the weights are
// found there again by the next step and are read with ordinary loads; larger ones only push other data out.
#define SWA_U 4
template <typename T, int HD, int NWAVES, bool STREAM = false>
__global__ void __launch_bounds__(NWAVES * 64)
swa_decode_kernel(const T* __restrict__ qkv, T* kring, T* vring, T* __restrict__ out, const float* __restrict__ slopes,
                  const int* __restrict__ dyn /* early in the list: within the preloaded argument dwords */, int H, int cap,
                  int pos, int window, float softcap, int append) {
  constexpr int DPL = HD / 8;
  constexpr int NGRP = NWAVES * 8;
  if (dyn) pos = dyn[0];
  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int grp = lane >> 3, gl = lane & 7;
  const int G = w * 8 + grp;
  const int d = H * HD;
  const T* row = qkv + (size_t)b * 3 * d + h * HD;
  const size_t hbase = ((size_t)b * H + h) * cap * HD;
  // the ring append: element `at` of the new key and value, read now by the last HD threads (no branch: the other
  // threads re-read element 0) and stored after everything else; slot pos % cap is not among the slots the sweep reads
  const int at = (int)threadIdx.x - (NWAVES * 64 - HD);
  const T app_k = row[d + max(at, 0)], app_v = row[2 * d + max(at, 0)];
  float q[DPL];
  load_pieces<T, DPL, false>(row, gl, q);
  const bool self_grp = append && (G == NGRP - 1);   // this group also takes the new token's own key
  // every group reads the new token's key and value (no branch, so nothing waits for them before the ring loads are
  // out); only the last group of the last wave gives them a weight
  float kself[DPL], vself[DPL];
  load_pieces<T, DPL, false>(row + d, gl, kself);
  load_pieces<T, DPL, false>(row + 2 * d, gl, vself);
  // Every wave keeps ONE running maximum for its 8 key groups (wave-wide max of the scores of an iteration), so the
  // groups of a wave merge by plain sums across lanes; only the NWAVES wave partials go through LDS.
  constexpr bool FAST = sizeof(T) == 2;
  const int lo = max(0, pos - window);
  const float scale = rsqrtf((float)HD), slope = slopes[h];
  const float inv_cap2l = softcap > 0.f ? 2.8853900817779268f / softcap : 0.f;
  const int j_end = append ? pos : pos + 1, slot_lo = lo % cap;
  const T* kb = kring + hbase;
  const T* vb = vring + hbase;
  float M = -INFINITY, l = 0.f, acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) acc[i] = 0.f;
  auto score = [&](const float* kk, int j) {
    float sc = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) sc = fmaf(q[i], kk[i], sc);
    sc = group8_sum(sc) * scale;
    if (softcap > 0.f) sc = soft_cap<FAST>(sc, softcap, inv_cap2l);
    return sc - slope * (float)(pos - j);
  };
  // wave-uniform loop: the wave's first group decides whether the wave has keys left
  for (int base = lo + w * 8 * SWA_U; base < j_end; base += NGRP * SWA_U) {
    const int jb = base + grp * SWA_U;
    float kk[SWA_U][DPL], vv[SWA_U][DPL];
    // no branch around the loads (a key beyond the range re-reads the last valid one and gets weight 0): all loads
    // of the iteration stay in flight together
#pragma unroll
    for (int u = 0; u < SWA_U; ++u) {
      const int j = min(jb + u, j_end - 1);
      int slot = slot_lo + (j - lo);
      slot = slot >= cap ? slot - cap : slot;
      load_pieces<T, DPL, STREAM>(kb + (size_t)slot * HD, gl, kk[u]);
      load_pieces<T, DPL, STREAM>(vb + (size_t)slot * HD, gl, vv[u]);
    }
    float sc[SWA_U], mit = -INFINITY;
#pragma unroll
    for (int u = 0; u < SWA_U; ++u) {
      const float v = score(kk[u], jb + u);
      sc[u] = (jb + u < j_end) ? v : -INFINITY;
      mit = fmaxf(mit, sc[u]);
    }
    const float Mn = fmaxf(M, wave_max(mit));     // finite: the wave's first key is valid
    const float corr = __expf(M - Mn);
    float psum = 0.f, p[SWA_U];
#pragma unroll
    for (int u = 0; u < SWA_U; ++u) { p[u] = __expf(sc[u] - Mn); psum += p[u]; }
    l = fmaf(l, corr, psum);
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      float a = acc[i] * corr;
#pragma unroll
      for (int u = 0; u < SWA_U; ++u) a = fmaf(p[u], vv[u][i], a);
      acc[i] = a;
    }
    M = Mn;
  }
  if (append && w == NWAVES - 1) {     // the new token's own key, taken by the last group of the last wave
    const float v = score(kself, pos);
    const float ss = self_grp ? v : -INFINITY;
    const float Mn = fmaxf(M, wave_max(ss));
    const float corr = __expf(M - Mn);
    const float ps = __expf(ss - Mn);
    l = fmaf(l, corr, ps);
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[i] = fmaf(ps, vself[i], acc[i] * corr);
    M = Mn;
  }
  // the wave's 8 groups share M: sums across the lanes 8, 16 and 32 apart
  auto xsum = [](float v) {
    v += fstu_dpp<0x128>(v);          // row_ror:8
    v += fstu_swz16(v);
    return v + __shfl_xor(v, 32, FSTU_WAVE);
  };
  l = xsum(l);
#pragma unroll
  for (int i = 0; i < DPL; ++i) acc[i] = xsum(acc[i]);
  __shared__ float wm[NWAVES], wl[NWAVES];
  __shared__ float wacc[NWAVES][HD];
  if (lane < 8) {
#pragma unroll
    for (int i = 0; i < DPL; ++i) wacc[w][piece_elem<T, DPL>(gl, i)] = acc[i];
    if (lane == 0) { wm[w] = M; wl[w] = l; }
  }
  __syncthreads();
  if (threadIdx.x < HD) {
    float M = -INFINITY;
#pragma unroll
    for (int g = 0; g < NWAVES; ++g) M = fmaxf(M, wm[g]);
    float Lsum = 0.f, o = 0.f;
#pragma unroll
    for (int g = 0; g < NWAVES; ++g) {
      const float e = (wm[g] == -INFINITY) ? 0.f : __expf(wm[g] - M);
      Lsum = fmaf(wl[g], e, Lsum);
      o = fmaf(wacc[g][threadIdx.x], e, o);
    }
    DT<T>::st(out + (size_t)b * d + h * HD + threadIdx.x, o / Lsum);
  }
  if (append && at >= 0) {
    const size_t dst = hbase + (size_t)(pos % cap) * HD + at;
    kring[dst] = app_k;
    vring[dst] = app_v;
  }
}

static int check_swa(const char* name, int H, int hd, int window, const void* slopes) {
  FSTU_REQUIRE(slopes, FSTU_ENULL, "%s: slopes is null", name);
  FSTU_REQUIRE(hd == 32 || hd == 64 || hd == 128 || hd == 256, FSTU_ESHAPE, "%s: head dim %d not in {32,64,128,256}", name, hd);
  FSTU_REQUIRE(window >= 0, FSTU_EARG, "%s: window<0", name);
  return FSTU_OK;
}

#define SWA_DISPATCH_HD(KERNEL, hd, ...)                                   \
  do {                                                                     \
    if (hd == 32) hipLaunchKernelGGL((KERNEL<T, 32>), __VA_ARGS__);        \
    else if (hd == 64) hipLaunchKernelGGL((KERNEL<T, 64>), __VA_ARGS__);   \
    else if (hd == 128) hipLaunchKernelGGL((KERNEL<T, 128>), __VA_ARGS__); \
    else hipLaunchKernelGGL((KERNEL<T, 256>), __VA_ARGS__);                \
  } while (0)

int fstu_swa_decode_impl(const void* qkv, void* kring, void* vring, void* out, const float* slopes, int B, int H, int hd,
                         int cap, int pos, int window, float softcap, int append, const int* dyn, int dtype, void* stream) {
  int rc = check_kv("fstu_swa_decode", qkv, kring, vring, B, H, hd, cap);
  if (rc) return rc;
  rc = check_swa("fstu_swa_decode", H, hd, window, slopes);
  if (rc) return rc;
  FSTU_REQUIRE(out, FSTU_ENULL, "fstu_swa_decode: out is null");
  FSTU_REQUIRE(pos >= 0 && cap >= window + 1, FSTU_EARG, "fstu_swa_decode: pos=%d, ring capacity %d < window+1=%d", pos, cap, window + 1);
  FSTU_REQUIRE(fstu_aligned(qkv, 16) && fstu_aligned(kring, 16) && fstu_aligned(vring, 16), FSTU_EALIGN, "fstu_swa_decode: pointers must be 16-byte aligned");
  FSTU_REQUIRE(B <= 65535, FSTU_ESHAPE, "fstu_swa_decode: B too large");
  hipStream_t s = (hipStream_t)stream;
  const int nkeys = dyn ? window + 1 : (pos < window ? pos : window) + 1;
  // keys and values one launch reads: from 64 MB on (a quarter of the memory-side cache) they are streamed
  const bool stream_ring = (size_t)B * H * nkeys * hd * 2 * (dtype == FSTU_BF16 ? 2 : 4) >= ((size_t)64 << 20);
#define SWA_LAUNCH(HD, NW)                                                                                              \
  do {                                                                                                                  \
    if (stream_ring)                                                                                                    \
      hipLaunchKernelGGL((swa_decode_kernel<T, HD, NW, true>), dim3(H, B), dim3(NW * 64), 0, s, (const T*)qkv, (T*)kring, \
                         (T*)vring, (T*)out, slopes, dyn, H, cap, pos, window, softcap, append);                        \
    else                                                                                                                \
      hipLaunchKernelGGL((swa_decode_kernel<T, HD, NW, false>), dim3(H, B), dim3(NW * 64), 0, s, (const T*)qkv, (T*)kring, \
                         (T*)vring, (T*)out, slopes, dyn, H, cap, pos, window, softcap, append);                        \
  } while (0)
  FSTU_DISPATCH_DTYPE(dtype, "fstu_swa_decode", {
    if (hd == 32) { if (nkeys > 128) SWA_LAUNCH(32, 16); else SWA_LAUNCH(32, 4); }
    // head dim 64, long windows: 8 waves (16 measured 1.5 us per decode step slower at window 512, 4 waves 3 us slower)
    else if (hd == 64) { if (nkeys > 128) SWA_LAUNCH(64, 8); else SWA_LAUNCH(64, 4); }
    else if (hd == 128) { if (nkeys > 128) SWA_LAUNCH(128, 8); else SWA_LAUNCH(128, 4); }
    else SWA_LAUNCH(256, 4);
  });
#undef SWA_LAUNCH
  FSTU_CHECK_LAUNCH("fstu_swa_decode");
  return FSTU_OK;
}

extern "C" int fstu_swa_decode(const void* qkv, const void* kring, const void* vring, void* out, const float* slopes,
                               int B, int H, int hd, int cap, int pos, int window, float softcap, int dtype,
                               void* stream) {
  return fstu_swa_decode_impl(qkv, (void*)kring, (void*)vring, out, slopes, B, H, hd, cap, pos, window, softcap, 0, nullptr, dtype, stream);
}

extern "C" int fstu_swa_append_decode(const void* qkv, void* kring, void* vring, void* out, const float* slopes, int B,
                                      int H, int hd, int cap, int pos, int window, float softcap, int dtype,
                                      void* stream) {
  return fstu_swa_decode_impl(qkv, kring, vring, out, slopes, B, H, hd, cap, pos, window, softcap, 1, nullptr, dtype, stream);
}

// ---------------------------------------------------------------- prefill
// One wave per (batch, head, query); 4 queries per workgroup.
template <typename T, int HD>
__global__ void __launch_bounds__(256)
swa_prefill_kernel(const T* __restrict__ qkv, T* __restrict__ out, const float* __restrict__ slopes, int Tn, int H,
                   int window, float softcap) {
  constexpr int DPL = HD / 8;
  __shared__ float sm[4][8], sl[4][8];
  __shared__ float sacc[4][8][HD];
  const int h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int grp = lane >> 3, gl = lane & 7;
  const int t = blockIdx.x * 4 + w;
  const int d = H * HD;
  const bool live = t < Tn;
  Partial<DPL> P;
  P.m = -INFINITY;
  P.l = 0.f;
#pragma unroll
  for (int i = 0; i < DPL; ++i) P.acc[i] = 0.f;
  if (live) {
    float q[DPL];
    const T* row0 = qkv + (size_t)b * Tn * 3 * d + h * HD + gl * DPL;
    load_vec<T, DPL>(row0 + (size_t)t * 3 * d, q);
    const int lo = max(0, t - window);
    attend_keys<T, DPL, SWA_U, sizeof(T) == 2>(P, row0 + d, row0 + 2 * d, (size_t)3 * d, 0, 0, 0, q, lo + grp * SWA_U, t + 1,
                                               8 * SWA_U, t, rsqrtf((float)HD), softcap, slopes[h]);
  }
  if (gl == 0) { sm[w][grp] = P.m; sl[w][grp] = P.l; }
#pragma unroll
  for (int i = 0; i < DPL; ++i) sacc[w][grp][gl * DPL + i] = P.acc[i];
  __syncthreads();
  if (live) {
    for (int i = lane; i < HD; i += 64) {
      float M = -INFINITY;
#pragma unroll
      for (int g = 0; g < 8; ++g) M = fmaxf(M, sm[w][g]);
      float Lsum = 0.f, o = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        float e = __expf(sm[w][g] - M);
        Lsum = fmaf(sl[w][g], e, Lsum);
        o = fmaf(sacc[w][g][i], e, o);
      }
      DT<T>::st(out + ((size_t)b * Tn + t) * d + h * HD + i, o / Lsum);
    }
  }
}

extern "C" int fstu_swa_prefill(const void* qkv, void* out, const float* slopes, int B, int T_, int H, int hd,
                                int window, float softcap, int dtype, void* stream) {
  FSTU_REQUIRE(qkv && out, FSTU_ENULL, "fstu_swa_prefill: null pointer");
  FSTU_REQUIRE(B >= 1 && T_ >= 1 && H >= 1 && B <= 65535 && H <= 65535, FSTU_ESHAPE, "fstu_swa_prefill: bad shape B=%d T=%d H=%d", B, T_, H);
  int rc = check_swa("fstu_swa_prefill", H, hd, window, slopes);
  if (rc) return rc;
  FSTU_REQUIRE(fstu_aligned(qkv, 16), FSTU_EALIGN, "fstu_swa_prefill: qkv must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  FSTU_DISPATCH_DTYPE(dtype, "fstu_swa_prefill",
                      SWA_DISPATCH_HD(swa_prefill_kernel, hd, dim3((T_ + 3) / 4, H, B), dim3(256), 0, s,
                                      (const T*)qkv, (T*)out, slopes, T_, H, window, softcap));
  FSTU_CHECK_LAUNCH("fstu_swa_prefill");
  return FSTU_OK;
}
