// Error reporting, embedding gather, fused residual + RMSNorm, GELU-gate and
// the sampling kernel.  All bandwidth-bound, one workgroup per row.
#include "fstu_common.h"
#include "fstu_prologue.h"
#include <string.h>

// ---------------------------------------------------------------- errors
static thread_local char g_err[512] = "";

void fstu_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* fstu_last_error(void) { return g_err; }
extern "C" int fstu_version(void) { return FSTU_VERSION; }

// ---------------------------------------------------------------- embed
template <typename T>
__global__ void embed_kernel(const int64_t* __restrict__ ids, int64_t id_stride, const T* __restrict__ table,
                             T* __restrict__ out, int d, int vocab, const int* __restrict__ dyn) {
  int r = blockIdx.x;
  int64_t id = ids[(size_t)r * id_stride + (dyn ? dyn[0] : 0)];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * d;
  T* dst = out + (size_t)r * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = src[i];
}

extern "C" int fstu_embed(const int64_t* ids, const void* table, void* out, int rows, int d, int vocab, int dtype,
                          void* stream) {
  FSTU_REQUIRE(ids && table && out, FSTU_ENULL, "fstu_embed: null pointer");
  FSTU_REQUIRE(rows >= 0 && d > 0 && vocab > 0, FSTU_ESHAPE, "fstu_embed: bad shape rows=%d d=%d vocab=%d", rows, d, vocab);
  if (rows == 0) return FSTU_OK;
  FSTU_DISPATCH_DTYPE(dtype, "fstu_embed",
                      hipLaunchKernelGGL(embed_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, ids,
                                         (int64_t)1, (const T*)table, (T*)out, d, vocab, (const int*)nullptr));
  FSTU_CHECK_LAUNCH("fstu_embed");
  return FSTU_OK;
}

// ids[r*id_stride (+ dyn[0])]: one column of a (rows, id_stride) token buffer (library-internal)
int fstu_embed_strided(const int64_t* ids, int64_t id_stride, const void* table, void* out, int rows, int d, int vocab,
                       int dtype, void* stream, const int* dyn) {
  FSTU_REQUIRE(ids && table && out, FSTU_ENULL, "fstu_embed: null pointer");
  FSTU_DISPATCH_DTYPE(dtype, "fstu_embed",
                      hipLaunchKernelGGL(embed_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, ids,
                                         id_stride, (const T*)table, (T*)out, d, vocab, dyn));
  FSTU_CHECK_LAUNCH("fstu_embed");
  return FSTU_OK;
}

// ---------------------------------------------------------------- add + rmsnorm
// One workgroup (256 threads) per row; a thread owns groups of 4 consecutive
// channels (16-byte fp32 loads, 8-byte bf16 loads) and keeps them in registers
// between the residual update and the normalisation.  Partial-sum slices are
// read four at a time into independent accumulators so their load latencies
// overlap; the summation order is fixed (deterministic).
#define FSTU_NORM_THREADS 256

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return s;
}

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  typedef float4 raw_t;
  static __device__ __forceinline__ raw_t ldraw(const float* p) { return *(const float4*)p; }
  static __device__ __forceinline__ void cvt(raw_t v, float* o) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
  static __device__ __forceinline__ void ld(const float* p, float* o) {
    float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
  static __device__ __forceinline__ void st(float* p, const float* v) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<bf16_t> {
  typedef uint2 raw_t;
  static __device__ __forceinline__ raw_t ldraw(const bf16_t* p) { return *(const uint2*)p; }
  static __device__ __forceinline__ void cvt(raw_t v, float* o) {
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void ld(const bf16_t* p, float* o) {
    uint2 v = *(const uint2*)p;
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float* v) {
    uint2 o;
    o.x = (unsigned)f32_to_bf16(v[0]) | ((unsigned)f32_to_bf16(v[1]) << 16);
    o.y = (unsigned)f32_to_bf16(v[2]) | ((unsigned)f32_to_bf16(v[3]) << 16);
    *(uint2*)p = o;
  }
};

// sum of `n` fp32 slices (stride `stride` floats) of 4 consecutive values in a fixed order; up to 16 slices are
// loaded before any is added so their latencies overlap
__device__ __forceinline__ void sum_slices4(const float* p, size_t stride, int n, float* out) {
  float4 tot = make_float4(0, 0, 0, 0);
  for (int s0 = 0; s0 < n; s0 += 16) {
    // no branch around the loads: a slice index beyond n re-reads the last slice and is added with weight 0
    float4 v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) v[k] = *(const float4*)(p + (size_t)min(s0 + k, n - 1) * stride);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float m = (s0 + k < n) ? 1.f : 0.f;
      tot.x = fmaf(m, v[k].x, tot.x); tot.y = fmaf(m, v[k].y, tot.y); tot.z = fmaf(m, v[k].z, tot.z); tot.w = fmaf(m, v[k].w, tot.w);
    }
  }
  out[0] = tot.x; out[1] = tot.y; out[2] = tot.z; out[3] = tot.w;
}

template <typename T, int NG, bool VEC>
__global__ void __launch_bounds__(FSTU_NORM_THREADS)
add_rmsnorm_kernel(T* __restrict__ x, const void* __restrict__ delta, int delta_mode, int nslices, int single_branch,
                   const T* __restrict__ w, T* __restrict__ y, int rows, int d, float eps) {
  // VEC: d % 4 == 0 and all pointers 16-byte aligned; a group is 4 channels.  Otherwise a group is 1 channel.
  constexpr int GW = VEC ? 4 : 1;
  __shared__ float red[4];
  const int r = blockIdx.x;
  T* xr = x + (size_t)r * d;
  const size_t slice = (size_t)rows * d;
  float v[NG][GW];
  // the norm weights are fetched up front: loaded after the row statistics they would add a second dependent
  // memory round trip to a kernel that is nothing but latency
  float wpre[NG][GW];
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (threadIdx.x + i * FSTU_NORM_THREADS) * GW;
    // no branch around the load (a branch with a zero on its other side makes the kernel wait for the load at once):
    // threads beyond the row re-read column 0, and without y the row itself stands in for the weights
    const T* wsrc = (y != nullptr) ? w : (const T*)xr;
    const int cw = c < d ? c : 0;
    if (VEC) Vec4<T>::ld(wsrc + cw, wpre[i]); else wpre[i][0] = DT<T>::ld(wsrc + cw);
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (threadIdx.x + i * FSTU_NORM_THREADS) * GW;
#pragma unroll
    for (int k = 0; k < GW; ++k) v[i][k] = 0.f;
    if (c < d) {
      float xv[GW], dv[GW];
      // the row is requested here and converted only after the delta loads are out: a conversion in between would
      // make the kernel wait for the row before it requests the slices
      typename Vec4<T>::raw_t xraw = {};
      T xraw1 = 0;
      if (VEC) xraw = Vec4<T>::ldraw(xr + c); else xraw1 = xr[c];
      if (delta != nullptr) {
        if (delta_mode == 0) {
          const T* dp = (const T*)delta + (size_t)r * d + c;
          if (VEC) Vec4<T>::ld(dp, dv); else dv[0] = DT<T>::ld(dp);
        } else if (delta_mode == 1) {
          const float* p = (const float*)delta + (size_t)r * d + c;
          if (VEC) {
            sum_slices4(p, slice, nslices, dv);
          } else {
            float acc = 0.f;
            for (int s = 0; s < nslices; ++s) acc += p[(size_t)s * slice];
            dv[0] = acc;
          }
#pragma unroll
          for (int k = 0; k < GW; ++k) dv[k] = DT<T>::rnd(dv[k]);
        } else {
          const float* p = (const float*)delta + (size_t)r * d + c;
          float e[GW], o[GW];
          if (VEC) {
            sum_slices4(p, 2 * slice, nslices, e);
            sum_slices4(p + slice, 2 * slice, nslices, o);
          } else {
            e[0] = o[0] = 0.f;
            for (int s = 0; s < nslices; ++s) { e[0] += p[(size_t)(2 * s) * slice]; o[0] += p[(size_t)(2 * s + 1) * slice]; }
          }
#pragma unroll
          for (int k = 0; k < GW; ++k)
            dv[k] = single_branch ? DT<T>::rnd(e[k] + o[k]) : DT<T>::rnd(DT<T>::rnd(e[k] + o[k]) + DT<T>::rnd(e[k] - o[k]));
        }
        if (VEC) Vec4<T>::cvt(xraw, xv); else xv[0] = DT<T>::ld(&xraw1);
#pragma unroll
        for (int k = 0; k < GW; ++k) xv[k] = DT<T>::rnd(xv[k] + dv[k]);
        if (VEC) Vec4<T>::st(xr + c, xv); else DT<T>::st(xr + c, xv[0]);
      } else {
        if (VEC) Vec4<T>::cvt(xraw, xv); else xv[0] = DT<T>::ld(&xraw1);
      }
#pragma unroll
      for (int k = 0; k < GW; ++k) { v[i][k] = xv[k]; ss += xv[k] * xv[k]; }
    }
  }
  if (y == nullptr) return;
  float tot = block_sum_256(ss, red);
  float rstd = rsqrtf(tot / (float)d + eps);
  T* yr = y + (size_t)r * d;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (threadIdx.x + i * FSTU_NORM_THREADS) * GW;
    if (c < d) {
      float o[GW];
#pragma unroll
      for (int k = 0; k < GW; ++k) o[k] = (v[i][k] * rstd) * wpre[i][k];
      if (VEC) Vec4<T>::st(yr + c, o); else DT<T>::st(yr + c, o[0]);
    }
  }
}

// Many rows (a prompt): one wave per row, four rows per workgroup, a lane owns chunks lane, lane+64, ... of 8 channels;
// no LDS and no barrier, every load of a row in flight at once.  Same arithmetic as add_rmsnorm_kernel with a
// model-dtype delta: x' = T(x + delta) written back, y = T((x' * rstd) * w).
__global__ void __launch_bounds__(256)
add_rmsnorm_rows_bf16_kernel(bf16_t* __restrict__ x, const bf16_t* __restrict__ delta, const bf16_t* __restrict__ w,
                             bf16_t* __restrict__ y, int rows, int d, float eps) {
  constexpr int NCH = 4;   // d <= 2048
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int nchunk = d >> 3;
  const fstu_rsrc_t rx = fstu_make_rsrc(x + (size_t)r * d, (size_t)d * 2);
  const fstu_rsrc_t rd = fstu_make_rsrc(delta ? delta + (size_t)r * d : nullptr, (size_t)d * 2);
  const fstu_rsrc_t rw = fstu_make_rsrc(y ? w : nullptr, (size_t)d * 2);
  uint4 xv[NCH], dv[NCH], wv[NCH];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const unsigned off = (unsigned)(lane + 64 * j) * 16u;   // beyond the row (or without the operand): zeros
    xv[j] = fstu_buf_load16(rx, off);
    dv[j] = fstu_buf_load16(rd, off);
    wv[j] = fstu_buf_load16(rw, off);
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    unsigned xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w};
    const unsigned dw[4] = {dv[j].x, dv[j].y, dv[j].z, dv[j].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (delta)
        xw[i] = pack2_bf16(__uint_as_float(xw[i] << 16) + __uint_as_float(dw[i] << 16),
                           __uint_as_float(xw[i] & 0xffff0000u) + __uint_as_float(dw[i] & 0xffff0000u));
      const float lo = __uint_as_float(xw[i] << 16), hi = __uint_as_float(xw[i] & 0xffff0000u);
      ss = fmaf(lo, lo, ss);
      ss = fmaf(hi, hi, ss);
    }
    xv[j] = make_uint4(xw[0], xw[1], xw[2], xw[3]);
    if (delta && lane + 64 * j < nchunk) *(uint4*)(x + (size_t)r * d + (size_t)(lane + 64 * j) * 8) = xv[j];
  }
  if (y == nullptr) return;
  const float rstd = rsqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    if (lane + 64 * j < nchunk) {
      const unsigned xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
      unsigned o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = pack2_bf16((__uint_as_float(xw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16),
                          (__uint_as_float(xw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u));
      *(uint4*)(y + (size_t)r * d + (size_t)(lane + 64 * j) * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

template <typename T>
static int launch_add_rmsnorm(void* x, const void* delta, int delta_mode, int nslices, int single_branch, const void* w,
                              void* y, int rows, int d, float eps, hipStream_t s) {
  if (sizeof(T) == 2 && rows >= 64 && (delta == nullptr || delta_mode == 0) && d % 8 == 0 && d <= 2048 &&
      fstu_aligned(x, 16) && fstu_aligned(delta, 16) && fstu_aligned(w, 16) && fstu_aligned(y, 16)) {
    hipLaunchKernelGGL(add_rmsnorm_rows_bf16_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)delta,
                       (const bf16_t*)w, (bf16_t*)y, rows, d, eps);
    return 0;
  }
  const bool vec = (d % 4 == 0) && fstu_aligned(x, 16) && fstu_aligned(delta, 16) && fstu_aligned(w, 16) && fstu_aligned(y, 16);
  const int groups = vec ? d / 4 : d;
  const int ng = (groups + FSTU_NORM_THREADS - 1) / FSTU_NORM_THREADS;
#define LAUNCH_NORM(NG, VEC)                                                                                          \
  hipLaunchKernelGGL((add_rmsnorm_kernel<T, NG, VEC>), dim3(rows), dim3(FSTU_NORM_THREADS), 0, s, (T*)x, delta,      \
                     delta_mode, nslices, single_branch, (const T*)w, (T*)y, rows, d, eps)
  if (vec) {
    if (ng <= 1) LAUNCH_NORM(1, true); else if (ng <= 2) LAUNCH_NORM(2, true); else if (ng <= 4) LAUNCH_NORM(4, true);
    else if (ng <= 8) LAUNCH_NORM(8, true); else return -1;
  } else {
    if (ng <= 4) LAUNCH_NORM(4, false); else if (ng <= 8) LAUNCH_NORM(8, false); else if (ng <= 32) LAUNCH_NORM(32, false);
    else return -1;
  }
#undef LAUNCH_NORM
  return 0;
}

// x = T(x + T(sum of nslices fp32 slices)) over rows*d elements, 4 per thread and 64 threads per workgroup, so that the
// few megabytes of slices are requested by the whole chip at once; the slices are added in the order fstu_add_rmsnorm
// uses (bit-identical x).  The rows' norm is left to the launch that consumes x.
__global__ void __launch_bounds__(64)
add_slices_bf16_kernel(bf16_t* __restrict__ x, const float* __restrict__ slices, int nslices, size_t n) {
  const size_t i4 = ((size_t)blockIdx.x * 64 + threadIdx.x) * 4;
  if (i4 >= n) return;
  const uint2 xr = *(const uint2*)(x + i4);
  float dv[4];
  sum_slices4(slices + i4, n, nslices, dv);
  const float x0 = __uint_as_float(xr.x << 16), x1 = __uint_as_float(xr.x & 0xffff0000u);
  const float x2 = __uint_as_float(xr.y << 16), x3 = __uint_as_float(xr.y & 0xffff0000u);
  *(uint2*)(x + i4) = make_uint2(pack2_bf16(x0 + DT<bf16_t>::rnd(dv[0]), x1 + DT<bf16_t>::rnd(dv[1])),
                                 pack2_bf16(x2 + DT<bf16_t>::rnd(dv[2]), x3 + DT<bf16_t>::rnd(dv[3])));
}

extern "C" int fstu_add_slices(void* x, const float* slices, int nslices, int rows, int d, int dtype, void* stream) {
  FSTU_REQUIRE(x && slices, FSTU_ENULL, "fstu_add_slices: null pointer");
  FSTU_REQUIRE(dtype == FSTU_BF16, FSTU_EDTYPE, "fstu_add_slices: bf16 only");
  FSTU_REQUIRE(rows >= 1 && d >= 4 && d % 4 == 0 && nslices >= 1, FSTU_ESHAPE, "fstu_add_slices: rows=%d d=%d nslices=%d", rows, d, nslices);
  FSTU_REQUIRE(fstu_aligned(x, 8) && fstu_aligned(slices, 16), FSTU_EALIGN, "fstu_add_slices: x must be 8-byte, slices 16-byte aligned");
  const size_t n = (size_t)rows * d;
  hipLaunchKernelGGL(add_slices_bf16_kernel, dim3((unsigned)((n / 4 + 63) / 64)), dim3(64), 0, (hipStream_t)stream, (bf16_t*)x, slices,
                     nslices, n);
  FSTU_CHECK_LAUNCH("fstu_add_slices");
  return FSTU_OK;
}

extern "C" int fstu_add_rmsnorm(void* x, const void* delta, int delta_mode, int nslices, int single_branch,
                                const void* w, void* y, int rows, int d, float eps, int dtype, void* stream) {
  FSTU_REQUIRE(x, FSTU_ENULL, "fstu_add_rmsnorm: x is null");
  FSTU_REQUIRE((y == nullptr) || (w != nullptr), FSTU_ENULL, "fstu_add_rmsnorm: y given without weight");
  FSTU_REQUIRE(delta || y, FSTU_EARG, "fstu_add_rmsnorm: nothing to do (no delta and no y)");
  FSTU_REQUIRE(rows >= 0 && d > 0 && d <= 8192, FSTU_ESHAPE, "fstu_add_rmsnorm: d=%d out of range (1..8192)", d);
  FSTU_REQUIRE(delta_mode >= 0 && delta_mode <= 2, FSTU_EARG, "fstu_add_rmsnorm: delta_mode=%d", delta_mode);
  FSTU_REQUIRE(delta == nullptr || delta_mode == 0 || nslices >= 1, FSTU_EARG, "fstu_add_rmsnorm: nslices=%d", nslices);
  if (rows == 0) return FSTU_OK;
  int rc;
  FSTU_DISPATCH_DTYPE(dtype, "fstu_add_rmsnorm",
                      rc = launch_add_rmsnorm<T>(x, delta, delta_mode, nslices, single_branch, w, y, rows, d, eps,
                                                 (hipStream_t)stream));
  FSTU_REQUIRE(rc == 0, FSTU_ESHAPE, "fstu_add_rmsnorm: d=%d not supported", d);
  FSTU_CHECK_LAUNCH("fstu_add_rmsnorm");
  return FSTU_OK;
}

// embedding gather fused with the first RMSNorm of the step: x[r,:] = table[id], h[r,:] = rmsnorm(x[r,:]) * w
template <typename T>
__global__ void __launch_bounds__(FSTU_NORM_THREADS)
embed_rmsnorm_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, T* __restrict__ x,
                     const T* __restrict__ w, T* __restrict__ h, const int* __restrict__ dyn, int64_t id_stride, int d,
                     int vocab, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  int64_t id = ids[(size_t)r * id_stride + (dyn ? dyn[0] : 0)];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * d;
  if (sizeof(T) == 2 && (d & 7) == 0 && d <= 8 * FSTU_NORM_THREADS &&
      (((uintptr_t)table | (uintptr_t)w | (uintptr_t)x | (uintptr_t)h) & 15) == 0) {
    // bf16 rows of up to 2048 channels: a thread owns one chunk of 8 channels; both loads sit in straight-line code
    // (a lane beyond the row reads zeros through the buffer descriptor), so one wait covers them
    const int nchunk = d >> 3, q = threadIdx.x;
    const uint4 wv4 = fstu_buf_load16(fstu_make_rsrc(w, (size_t)d * 2), (unsigned)q * 16u);
    const uint4 xv4 = fstu_buf_load16(fstu_make_rsrc(src, (size_t)d * 2), (unsigned)q * 16u);
    const unsigned xw[4] = {xv4.x, xv4.y, xv4.z, xv4.w}, ww[4] = {wv4.x, wv4.y, wv4.z, wv4.w};
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = __uint_as_float(xw[i] << 16), hi = __uint_as_float(xw[i] & 0xffff0000u);
      ss = fmaf(lo, lo, ss);
      ss = fmaf(hi, hi, ss);
    }
    if (q < nchunk) *(uint4*)((bf16_t*)x + (size_t)r * d + q * 8) = xv4;
    const float rstd = rsqrtf(block_sum_256(ss, red) / (float)d + eps);
    if (q < nchunk) {
      unsigned o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = pack2_bf16((__uint_as_float(xw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16),
                          (__uint_as_float(xw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u));
      *(uint4*)((bf16_t*)h + (size_t)r * d + q * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
    return;
  }
  // norm weights and the embedding row are both read before the reduction (up to 8 columns per thread stay in
  // registers), so that nothing is fetched after it
  constexpr int PRE = 8;
  float wv[PRE], xv[PRE];
#pragma unroll
  for (int k = 0; k < PRE; ++k) {
    const int c = threadIdx.x + k * FSTU_NORM_THREADS;
    wv[k] = (c < d) ? DT<T>::ld(w + c) : 0.f;
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < PRE; ++k) {
    const int c = threadIdx.x + k * FSTU_NORM_THREADS;
    xv[k] = 0.f;
    if (c < d) {
      T raw = src[c];
      x[(size_t)r * d + c] = raw;
      xv[k] = DT<T>::ld(&raw);
      ss = fmaf(xv[k], xv[k], ss);
    }
  }
  for (int c = threadIdx.x + PRE * FSTU_NORM_THREADS; c < d; c += FSTU_NORM_THREADS) {
    T raw = src[c];
    x[(size_t)r * d + c] = raw;
    float v = DT<T>::ld(&raw);
    ss = fmaf(v, v, ss);
  }
  const float rstd = rsqrtf(block_sum_256(ss, red) / (float)d + eps);
#pragma unroll
  for (int k = 0; k < PRE; ++k) {
    const int c = threadIdx.x + k * FSTU_NORM_THREADS;
    if (c < d) DT<T>::st(h + (size_t)r * d + c, (xv[k] * rstd) * wv[k]);
  }
  for (int c = threadIdx.x + PRE * FSTU_NORM_THREADS; c < d; c += FSTU_NORM_THREADS)
    DT<T>::st(h + (size_t)r * d + c, (DT<T>::ld(src + c) * rstd) * DT<T>::ld(w + c));
}

int fstu_embed_rmsnorm(const int64_t* ids, int64_t id_stride, const void* table, void* x, const void* w, void* h, int rows,
                       int d, int vocab, float eps, int dtype, void* stream, const int* dyn) {
  FSTU_REQUIRE(ids && table && x && w && h, FSTU_ENULL, "fstu_embed_rmsnorm: null pointer");
  FSTU_DISPATCH_DTYPE(dtype, "fstu_embed_rmsnorm",
                      hipLaunchKernelGGL(embed_rmsnorm_kernel<T>, dim3(rows), dim3(FSTU_NORM_THREADS), 0, (hipStream_t)stream,
                                         ids, (const T*)table, (T*)x, (const T*)w, (T*)h, dyn, id_stride, d, vocab, eps));
  FSTU_CHECK_LAUNCH("fstu_embed_rmsnorm");
  return FSTU_OK;
}

// ---------------------------------------------------------------- greedy pick of one step finished inside the next step's first launch
// The head of a greedy step leaves 64 packed maxima per row ((key << 32) | ~index).  Inside a graph of several steps the
// launch that would reduce them, store the token and advance the device-side position is followed at once by the
// next step's embedding + norm launch, which needs nothing but that token: both are one launch here.  One
// workgroup, one wave per row (so the position is read by every wave before thread 0 advances it); a lane owns
// chunks lane, lane+64, ... (8 channels each) of its row.
__global__ void __launch_bounds__(1024)
finish_embed_rmsnorm_kernel(unsigned long long* __restrict__ best, int64_t* __restrict__ tok_out, int64_t stride,
                            const bf16_t* __restrict__ table, bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                            bf16_t* __restrict__ h, int* __restrict__ dyn, int d, int vocab, float eps) {
  constexpr int NCH = 4;   // d <= 2048
  const int b = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = dyn[0];
  unsigned long long k = best[(size_t)b * 64 + lane];
  uint4 wv[NCH], xv[NCH];
  const fstu_rsrc_t rw = fstu_make_rsrc(w, (size_t)d * 2);
#pragma unroll
  for (int j = 0; j < NCH; ++j) wv[j] = fstu_buf_load16(rw, (unsigned)(lane + 64 * j) * 16u);
  best[(size_t)b * 64 + lane] = 0ull;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    unsigned long long t = __shfl_xor(k, o, FSTU_WAVE);
    k = t > k ? t : k;
  }
  int64_t id = (int64_t)(0xffffffffu - (unsigned)(k & 0xffffffffull));
  __syncthreads();
  if (threadIdx.x == 0) { dyn[0] = pos + 1; dyn[1] += 1; }
  if (lane == 0) tok_out[(size_t)b * stride + pos] = id;
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const fstu_rsrc_t rx = fstu_make_rsrc(table + (size_t)id * d, (size_t)d * 2);
#pragma unroll
  for (int j = 0; j < NCH; ++j) xv[j] = fstu_buf_load16(rx, (unsigned)(lane + 64 * j) * 16u);
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const unsigned xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = __uint_as_float(xw[i] << 16), hi = __uint_as_float(xw[i] & 0xffff0000u);
      ss = fmaf(lo, lo, ss);
      ss = fmaf(hi, hi, ss);
    }
  }
  const float rstd = rsqrtf(wave_sum(ss) / (float)d + eps);
  const int nchunk = d >> 3;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int q = lane + 64 * j;
    if (q < nchunk) {
      const unsigned xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
      unsigned o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = pack2_bf16((__uint_as_float(xw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16),
                          (__uint_as_float(xw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u));
      *(uint4*)(x + (size_t)b * d + q * 8) = xv[j];
      *(uint4*)(h + (size_t)b * d + q * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

bool fstu_finish_embed_supported(int rows, int d, const void* table, const void* x, const void* w, const void* h) {
  return rows >= 1 && rows <= 16 && (d & 7) == 0 && d <= 2048 &&
         (((uintptr_t)table | (uintptr_t)w | (uintptr_t)x | (uintptr_t)h) & 15) == 0;
}

int fstu_finish_embed_rmsnorm(void* best_ws, int64_t* tok_out, int64_t tok_stride, const void* table, void* x, const void* w,
                              void* h, int* dyn, int rows, int d, int vocab, float eps, void* stream) {
  FSTU_REQUIRE(best_ws && tok_out && table && x && w && h && dyn, FSTU_ENULL, "fstu_finish_embed_rmsnorm: null pointer");
  FSTU_REQUIRE(fstu_finish_embed_supported(rows, d, table, x, w, h), FSTU_ESHAPE,
               "fstu_finish_embed_rmsnorm: rows=%d d=%d unsupported (rows <= 16, d %% 8 == 0, d <= 2048, 16-byte aligned)", rows, d);
  hipLaunchKernelGGL(finish_embed_rmsnorm_kernel, dim3(1), dim3(rows * 64), 0, (hipStream_t)stream,
                     (unsigned long long*)best_ws, tok_out, tok_stride, (const bf16_t*)table, (bf16_t*)x, (const bf16_t*)w,
                     (bf16_t*)h, dyn, d, vocab, eps);
  FSTU_CHECK_LAUNCH("fstu_finish_embed_rmsnorm");
  return FSTU_OK;
}

// ---------------------------------------------------------------- gelu * up
template <typename T>
__global__ void gelu_mul_kernel(const T* __restrict__ g, const T* __restrict__ u, T* __restrict__ act, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float ge = DT<T>::rnd(gelu_tanh_f32(DT<T>::ld(g + i)));
    DT<T>::st(act + i, ge * DT<T>::ld(u + i));
  }
}

// bf16, 8 elements (16 bytes) per thread and iteration
__global__ void __launch_bounds__(256)
gelu_mul_bf16x8_kernel(const uint4* __restrict__ g, const uint4* __restrict__ u, uint4* __restrict__ act, int64_t n8) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n8; i += stride) {
    const uint4 gv = g[i], uv = u[i];
    unsigned gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w}, ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float lo = DT<bf16_t>::rnd(gelu_tanh_f32(__uint_as_float(gw[k] << 16))) * __uint_as_float(uw[k] << 16);
      float hi = DT<bf16_t>::rnd(gelu_tanh_f32(__uint_as_float(gw[k] & 0xffff0000u))) * __uint_as_float(uw[k] & 0xffff0000u);
      ow[k] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
    }
    act[i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

extern "C" int fstu_gelu_mul(const void* g, const void* u, void* act, int64_t n, int dtype, void* stream) {
  FSTU_REQUIRE(g && u && act, FSTU_ENULL, "fstu_gelu_mul: null pointer");
  FSTU_REQUIRE(n >= 0, FSTU_ESHAPE, "fstu_gelu_mul: n<0");
  if (n == 0) return FSTU_OK;
  if (dtype == FSTU_BF16 && n % 8 == 0 && fstu_aligned(g, 16) && fstu_aligned(u, 16) && fstu_aligned(act, 16)) {
    int64_t b8 = (n / 8 + 255) / 256;
    if (b8 > 16384) b8 = 16384;
    hipLaunchKernelGGL(gelu_mul_bf16x8_kernel, dim3((unsigned)b8), dim3(256), 0, (hipStream_t)stream, (const uint4*)g,
                       (const uint4*)u, (uint4*)act, n / 8);
    FSTU_CHECK_LAUNCH("fstu_gelu_mul");
    return FSTU_OK;
  }
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  FSTU_DISPATCH_DTYPE(dtype, "fstu_gelu_mul",
                      hipLaunchKernelGGL(gelu_mul_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                                         (const T*)g, (const T*)u, (T*)act, n));
  FSTU_CHECK_LAUNCH("fstu_gelu_mul");
  return FSTU_OK;
}

// ---------------------------------------------------------------- bias + activation
// y[r,c] = act( T(y[r,c] + bias[c]) ), act = identity or x*sigmoid(x); bias may be null
template <typename T>
__global__ void bias_act_kernel(T* __restrict__ y, const T* __restrict__ bias, int64_t rows, int n, int kind) {
  const int64_t total = rows * n;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    float v = DT<T>::ld(y + i);
    if (bias) v = DT<T>::rnd(v + DT<T>::ld(bias + (i % n)));
    if (kind == 1) v = v / (1.0f + expf(-v));
    DT<T>::st(y + i, v);
  }
}

extern "C" int fstu_bias_act(void* y, const void* bias, int64_t rows, int n, int kind, int dtype, void* stream) {
  FSTU_REQUIRE(y, FSTU_ENULL, "fstu_bias_act: null pointer");
  FSTU_REQUIRE(rows >= 0 && n >= 1 && (kind == 0 || kind == 1), FSTU_EARG, "fstu_bias_act: rows=%lld n=%d kind=%d", (long long)rows, n, kind);
  if (rows == 0 || (!bias && kind == 0)) return FSTU_OK;
  int64_t blocks = (rows * n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  FSTU_DISPATCH_DTYPE(dtype, "fstu_bias_act",
                      hipLaunchKernelGGL(bias_act_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                                         (T*)y, (const T*)bias, rows, n, kind));
  FSTU_CHECK_LAUNCH("fstu_bias_act");
  return FSTU_OK;
}

// ---------------------------------------------------------------- sampling
// One workgroup of 1024 threads per row; the row (V logits) is re-read from
// L2 in each pass instead of being staged.

struct SampleShared {
  float redf[16];
  int redi[16];
  double redd[16];
  unsigned hist[256];
  unsigned long long mass[256];
  unsigned sel_prefix;
  unsigned sel_k;
  unsigned long long sel_mass;
  int bcast_i;
  double bcast_d;
};

__device__ __forceinline__ unsigned f32_key(float f) {  // larger float -> larger key
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_f32(unsigned k) {
  unsigned u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

template <typename T>
__device__ __forceinline__ float sample_transform(const T* row, int i, float inv_temp_is_one, float temperature) {
  float x = DT<T>::ld(row + i);
  if (!inv_temp_is_one) x = DT<T>::rnd(x / temperature);
  x = fminf(fmaxf(x, -1e4f), 1e4f);
  return DT<T>::rnd(x);
}

template <int NT>
__device__ __forceinline__ double block_excl_scan_d(double v, double* red, double* total) {
  // exclusive scan over NT threads (NT/64 <= 16 waves), fixed order
  int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  double inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    double t = __shfl_up(inc, o, FSTU_WAVE);
    if (lane >= o) inc += t;
  }
  if (lane == 63) red[w] = inc;
  __syncthreads();
  double base = 0.0, tot = 0.0;
  for (int i = 0; i < NT / 64; ++i) {
    if (i < w) base += red[i];
    tot += red[i];
  }
  __syncthreads();
  *total = tot;
  return base + inc - v;
}

// Bin selection of a radix-select pass by wave 0 (every lane of that wave calls it): the highest bin b with
// base + (sum of the bins above b) + h[b] >= need (STRICT: > need), bin 0 if there is none; *above_out receives
// base + the sum of the bins above the selected one.  Lane l owns bins 4l .. 4l+3; the sums over higher lanes come
// from a suffix scan across the wave instead of one thread walking 256 LDS words.
template <typename C, bool STRICT>
__device__ __forceinline__ int select_bin_wave0(const C* h, C base, C need, C* above_out) {
  const int lane = threadIdx.x & 63;
  C v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = h[lane * 4 + j];
  const C mine = v[0] + v[1] + v[2] + v[3];
  C suf = mine;                                   // inclusive suffix sum over lanes >= lane
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const C t = __shfl_down(suf, o, FSTU_WAVE);
    if (lane + o < 64) suf += t;
  }
  C ab = base + (suf - mine);                     // bins above this lane's highest bin
  int found = -1;
  C found_above = 0;
#pragma unroll
  for (int j = 3; j >= 0; --j) {
    const bool hit = STRICT ? (ab + v[j] > need) : (ab + v[j] >= need);
    if (found < 0 && hit) { found = lane * 4 + j; found_above = ab; }
    ab += v[j];
  }
  const unsigned long long any = __ballot(found >= 0);
  if (any == 0ull) {                              // no bin reaches it: bin 0, everything above bin 0
    const C tot = __shfl(suf, 0, FSTU_WAVE);      // lane 0's inclusive suffix = all bins
    const C h0 = __shfl(v[0], 0, FSTU_WAVE);
    *above_out = base + tot - h0;
    return 0;
  }
  const int top = 63 - __clzll((long long)any);   // the highest lane with a hit holds the highest bin
  *above_out = __shfl(found_above, top, FSTU_WAVE);
  return __shfl(found, top, FSTU_WAVE);
}

// CACHE (16-bit dtypes, rows of up to 64 K logits): the first pass leaves the transformed logits (temperature, clamp,
// rounding: themselves 16-bit values) in LDS and every later pass reads them there instead of repeating the
// division per element from L2.
// One row by the NT threads of a workgroup; the picked token goes to *out_slot.
template <typename T, bool CACHE, int NT>
__device__ __forceinline__ void sample_row(SampleShared& sh, unsigned short* tl /*CACHE: V 16-bit words of LDS*/,
                                           const T* __restrict__ row, int64_t* __restrict__ out_slot, int V, float temperature,
                                           int top_k, float top_p, int do_sample, uint64_t seed, int step, int rowid) {
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const bool t1 = (temperature == 1.0f);
  auto tv = [&](int i) -> float {
    return CACHE ? __uint_as_float((unsigned)tl[i] << 16) : sample_transform(row, i, t1, temperature);
  };

  // ---- pass A: maximum (lowest index on ties) over a strided walk
  float best = -INFINITY;
  int besti = 0x7fffffff;
  {
    // 8 strided loads in flight per thread; indices grow with k, so '>' keeps the lowest index on ties
    int i = tid;
    for (; i + 7 * NT < V; i += 8 * NT) {
      float l[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        l[k] = sample_transform(row, i + k * NT, t1, temperature);
        if (CACHE) tl[i + k * NT] = (unsigned short)(__float_as_uint(l[k]) >> 16);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (besti == 0x7fffffff || l[k] > best) { best = l[k]; besti = i + k * NT; }
    }
    for (; i < V; i += NT) {
      float l = sample_transform(row, i, t1, temperature);
      if (CACHE) tl[i] = (unsigned short)(__float_as_uint(l) >> 16);
      if (besti == 0x7fffffff || l > best) { best = l; besti = i; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ob = __shfl_xor(best, o, FSTU_WAVE);
    int oi = __shfl_xor(besti, o, FSTU_WAVE);
    if (ob > best || (ob == best && oi < besti)) { best = ob; besti = oi; }
  }
  if (lane == 0) { sh.redf[w] = best; sh.redi[w] = besti; }
  __syncthreads();
  if (tid == 0) {
    float bb = sh.redf[0];
    int bi = sh.redi[0];
    for (int i = 1; i < NT / 64; ++i)
      if (sh.redf[i] > bb || (sh.redf[i] == bb && sh.redi[i] < bi)) { bb = sh.redf[i]; bi = sh.redi[i]; }
    sh.redf[0] = bb;
    sh.bcast_i = bi;
  }
  __syncthreads();
  const float m = sh.redf[0];
  const int arg = sh.bcast_i;
  __syncthreads();
  if (!do_sample) {
    if (tid == 0) *out_slot = arg;
    return;
  }

  // A 16-bit model dtype leaves the low 16 bits of every key the same for a given leading half (zeros for positive
  // values, ones for negative ones, whose keys are complemented): the two low radix passes would find all their
  // candidates in one bin, so they are skipped and the low half is filled in.
  constexpr int LOW_SHIFT = sizeof(T) == 2 ? 16 : 0;
  auto low_bits = [](unsigned prefix) -> unsigned {
    return sizeof(T) == 2 ? ((prefix & 0x80000000u) ? 0u : 0xffffu) : 0u;
  };
  // ---- top-k threshold by radix select on the monotone key
  unsigned thr_key = 0;  // keep keys >= thr_key
  if (top_k > 0 && top_k < V) {
    unsigned prefix = 0, kk = (unsigned)top_k;
    for (int shift = 24; shift >= LOW_SHIFT; shift -= 8) {
      for (int i = tid; i < 256; i += NT) sh.hist[i] = 0;
      __syncthreads();
      unsigned himask = (shift == 24) ? 0u : (0xffffffffu << (shift + 8));
      // 8 strided loads in flight per thread (one load per trip would make every trip a round trip to the L2)
      for (int i0 = tid; i0 < V; i0 += 8 * NT) {
        unsigned k[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) k[u] = f32_key(tv(min(i0 + u * NT, V - 1)));
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (i0 + u * NT < V && (k[u] & himask) == (prefix & himask)) atomicAdd(&sh.hist[(k[u] >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (w == 0) {
        unsigned acc;
        const int bin = select_bin_wave0<unsigned, false>(sh.hist, 0u, kk, &acc);
        if (tid == 0) {
          sh.sel_prefix = prefix | ((unsigned)bin << shift);
          sh.sel_k = kk - acc;
        }
      }
      __syncthreads();
      prefix = sh.sel_prefix;
      kk = sh.sel_k;
      __syncthreads();
    }
    thr_key = prefix | low_bits(prefix);
  }

  // ---- top-p over the survivors
  // kept set = {key > vb} U {key == vb with tie rank < tie_keep}
  unsigned vb_key = thr_key;
  long long tie_keep = -1;  // -1: keep every tied token
  if (top_p > 0.f && top_p < 1.f) {
    double e = 0.0;
    // (sums stay in index order per thread: the batches only put 8 loads in flight together)
    for (int i0 = tid; i0 < V; i0 += 8 * NT) {
      float l[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) l[u] = tv(min(i0 + u * NT, V - 1));
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (i0 + u * NT < V && f32_key(l[u]) >= thr_key) e += (double)expf(l[u] - m);
    }
    double Z1;
    block_excl_scan_d<NT>(e, sh.redd, &Z1);
    const double scale = 17592186044416.0 / Z1;  // 2^44 / Z1: fixed-point probabilities
    const unsigned long long target = (unsigned long long)((double)top_p * 17592186044416.0);
    unsigned prefix = 0;
    unsigned long long above = 0;  // mass of keys strictly above the current prefix range
    for (int shift = 24; shift >= LOW_SHIFT; shift -= 8) {
      for (int i = tid; i < 256; i += NT) sh.mass[i] = 0ull;
      __syncthreads();
      unsigned himask = (shift == 24) ? 0u : (0xffffffffu << (shift + 8));
      for (int i0 = tid; i0 < V; i0 += 8 * NT) {
        float l[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) l[u] = tv(min(i0 + u * NT, V - 1));
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const unsigned k = f32_key(l[u]);
          if (i0 + u * NT < V && k >= thr_key && (k & himask) == (prefix & himask))
            atomicAdd(&sh.mass[(k >> shift) & 255u], (unsigned long long)((double)expf(l[u] - m) * scale));
        }
      }
      __syncthreads();
      if (w == 0) {
        // lowest bin whose strictly-above mass is still <= target (bins below it have mass-above > target)
        unsigned long long acc;
        const int bin = select_bin_wave0<unsigned long long, true>(sh.mass, above, target, &acc);
        if (tid == 0) {
          sh.sel_prefix = prefix | ((unsigned)bin << shift);
          sh.sel_mass = acc;
        }
      }
      __syncthreads();
      prefix = sh.sel_prefix;
      above = sh.sel_mass;
      __syncthreads();
    }
    prefix |= low_bits(prefix);
    // prefix = boundary key vb: mass strictly above it is `above` (<= target);
    // tokens tied at vb are kept while above + rank*p_b <= target.
    if (prefix >= thr_key) {
      vb_key = prefix;
      float lb = key_f32(vb_key);
      unsigned long long pb = (unsigned long long)((double)expf(lb - m) * scale);
      if (pb == 0ull) pb = 1ull;
      tie_keep = (long long)((target - above) / pb) + 1;  // above <= target by construction
    }  // else: top-p keeps every top-k survivor
  }

  // ---- draw: inverse CDF in index order over contiguous per-thread chunks
  const int chunk = (V + NT - 1) / NT;
  const int i0 = tid * chunk, i1 = min(V, i0 + chunk);
  // tie ranks need an index-ordered count of tokens equal to vb
  double tcount = 0.0;
  if (tie_keep >= 0)
    for (int i = i0; i < i1; ++i)
      if (f32_key(tv(i)) == vb_key) tcount += 1.0;
  double ttotal = 0.0;
  double tbase = (tie_keep >= 0) ? block_excl_scan_d<NT>(tcount, sh.redd, &ttotal) : 0.0;
  double mysum = 0.0;
  {
    long long rank = (long long)tbase;
    for (int i = i0; i < i1; ++i) {
      float l = tv(i);
      unsigned k = f32_key(l);
      bool keep = k > vb_key;
      if (k == vb_key) { keep = (tie_keep < 0) || (rank < tie_keep); ++rank; }
      if (keep) mysum += (double)expf(l - m);
    }
  }
  double Z;
  double mybase = block_excl_scan_d<NT>(mysum, sh.redd, &Z);
  // counter-based uniform (splitmix64 finaliser), 24 bits
  unsigned long long z = seed * 0x9E3779B97F4A7C15ull + (unsigned long long)step * 0xBF58476D1CE4E5B9ull +
                         (unsigned long long)rowid * 0x94D049BB133111EBull + 0x2545F4914F6CDD1Dull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  const double u = (double)(z >> 40) / 16777216.0;
  const double tgt = u * Z;
  if (tid == 0) sh.bcast_i = -1;
  __syncthreads();
  if (mysum > 0.0 && tgt >= mybase && tgt < mybase + mysum) {
    double acc = mybase;
    long long rank = (long long)tbase;
    int pick = -1, lastkept = -1;
    for (int i = i0; i < i1; ++i) {
      float l = tv(i);
      unsigned k = f32_key(l);
      bool keep = k > vb_key;
      if (k == vb_key) { keep = (tie_keep < 0) || (rank < tie_keep); ++rank; }
      if (keep) {
        acc += (double)expf(l - m);
        lastkept = i;
        if (acc > tgt) { pick = i; break; }
      }
    }
    if (pick < 0) pick = lastkept;
    sh.bcast_i = pick;
  }
  __syncthreads();
  if (tid == 0) {
    int pick = sh.bcast_i;
    if (pick < 0) pick = arg;  // rounding left the target past the last chunk
    *out_slot = pick;
  }
}

#define FSTU_SAMPLE_THREADS 1024
template <typename T, bool CACHE>
__global__ void __launch_bounds__(FSTU_SAMPLE_THREADS)
sample_kernel(const T* __restrict__ logits, int64_t* __restrict__ out, int64_t out_stride, int V, float temperature,
              int top_k, float top_p, int do_sample, uint64_t seed, int step, int row0, const int* __restrict__ dyn) {
  __shared__ SampleShared sh;
  extern __shared__ unsigned short tl[];   // CACHE: transformed logits of the row
  const int b = blockIdx.x;
  if (dyn) { out += dyn[0]; step = dyn[1]; }
  sample_row<T, CACHE, FSTU_SAMPLE_THREADS>(sh, tl, logits + (size_t)b * V, out + (size_t)b * out_stride, V, temperature, top_k,
                                            top_p, do_sample, seed, step, b + row0);
}

// ---------------------------------------------------------------- top-k sampling across the chip
// The same draw as sample_row for 1 <= top_k <= 64 on 16-bit logits, in one launch of (V / 2048) x B workgroups
// instead of one workgroup per row (reference: flash_stu/model.py:267-299).
//
// The head kernel leaves, per row, the maxima of 64 disjoint subsets of the vocabulary (the packed slots of its
// greedy pick, already temperature-scaled): the top_k-th largest of them is a lower bound Lb of the row's top_k-th
// largest logit, because top_k different tokens reach it.  Every workgroup transforms one chunk of 2048 logits (one
// 16-byte load per thread) and leaves the few tokens >= Lb (about 60 of 50 K at top_k 40) in its own part of a
// workspace, in index order.  The last workgroup of a row to finish (a ticket per row) collects them and one wave
// does the rest on that short list: exact threshold, optional top-p, inverse-CDF draw in index order, with the
// arithmetic of sample_row.  A chunk with more than SAMP_CHUNK_CAP candidates (plateaus of equal logits) makes the
// last workgroup run sample_row on the whole row instead, so every input has an answer.  The counters of the workspace
// and the slots are zero on entry and zero again on exit; with `advance` the last workgroup of the launch bumps
// {pos, step}.
#define SAMP_CHUNK 2048
#define SAMP_CHUNK_CAP 32
#define SAMP_MAX_CHUNKS 32
#define SAMP_MAX_ROWS (2 * FSTU_MAX_DECODE_ROWS)
struct SampWs {
  unsigned ticket[SAMP_MAX_ROWS][32];   // one 128-byte line per row: atomics on one line are served one after the other
  unsigned done;
  unsigned pad[31];
  unsigned cnt[SAMP_MAX_ROWS][SAMP_MAX_CHUNKS];
  unsigned cand[SAMP_MAX_ROWS][SAMP_MAX_CHUNKS][SAMP_CHUNK_CAP];   // (index << 16) | 16-bit key
};

// exchanged between workgroups on different XCDs: agent-scope accesses, which the per-XCD L2 does not keep stale
__device__ __forceinline__ void st_agent(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned ld_agent(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// value of a 16-bit key (the upper half of f32_key of a 16-bit float)
__device__ __forceinline__ float key16_f32(unsigned k16) {
  return key_f32((k16 << 16) | ((k16 & 0x8000u) ? 0u : 0xffffu));
}

__global__ void __launch_bounds__(256)
sample_topk_kernel(const bf16_t* __restrict__ logits, int64_t ldl, unsigned long long* __restrict__ best,
                   SampWs* __restrict__ ws, int64_t* __restrict__ out, int64_t out_stride, int V, float temperature, int top_k,
                   float top_p, uint64_t seed, int step, int row0, int* __restrict__ dyn, int advance) {
  __shared__ SampleShared sh;
  __shared__ int s_wtot[4], s_last, s_n, s_over;
  __shared__ int s_off[SAMP_MAX_CHUNKS + 1];
  __shared__ unsigned short c_idx[SAMP_MAX_CHUNKS * SAMP_CHUNK_CAP], c_key[SAMP_MAX_CHUNKS * SAMP_CHUNK_CAP];
  __shared__ float c_e[SAMP_MAX_CHUNKS * SAMP_CHUNK_CAP];
  __shared__ unsigned long long c_mass[SAMP_MAX_CHUNKS * SAMP_CHUNK_CAP];
  const int b = blockIdx.y, g = blockIdx.x, G = gridDim.x, nrows = gridDim.y;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  int pos_off = 0;
  if (dyn) { pos_off = dyn[0]; step = dyn[1]; }
  const bf16_t* row = logits + (size_t)b * ldl;
  const unsigned long long slot = best[(size_t)b * 64 + lane];   // every wave: the row's 64 slot maxima
  // this thread's 8 logits (the row's last vector is moved back inside the row; its first elements then belong to
  // the thread before and are masked here)
  const int v0 = (g * 256 + tid) * 8;
  const int e0 = min(v0, V - 8);
  uint4 raw;
  __builtin_memcpy(&raw, row + e0, 16);   // rows start at any even address
  const unsigned sk = (unsigned)(slot >> 48);
  unsigned Lb = 0;
#pragma unroll
  for (int bit = 15; bit >= 0; --bit) {
    const unsigned cnd = Lb | (1u << bit);
    if (__popcll(__ballot(sk >= cnd)) >= top_k) Lb = cnd;
  }
  const bool t1 = temperature == 1.0f;
  const unsigned rw[4] = {raw.x, raw.y, raw.z, raw.w};
  unsigned keys[8], mask = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float x = __uint_as_float((j & 1) ? (rw[j >> 1] & 0xffff0000u) : (rw[j >> 1] << 16));
    if (!t1) x = DT<bf16_t>::rnd(x / temperature);
    x = DT<bf16_t>::rnd(fminf(fmaxf(x, -1e4f), 1e4f));
    keys[j] = f32_key(x) >> 16;
    if (e0 + j >= v0 && v0 < V && keys[j] >= Lb) mask |= 1u << j;
  }
  // candidates in index order: thread order, then element order
  const int mine = __popc(mask);
  int inc = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(inc, o, FSTU_WAVE);
    if (lane >= o) inc += t;
  }
  if (lane == 63) s_wtot[w] = inc;
  __syncthreads();
  int at = inc - mine, tot = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i < w) at += s_wtot[i];
    tot += s_wtot[i];
  }
  unsigned* dst = ws->cand[b][g];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if ((mask >> j) & 1u) {
      if (at < SAMP_CHUNK_CAP) st_agent(dst + at, ((unsigned)(e0 + j) << 16) | keys[j]);
      ++at;
    }
  if (tid == 0) st_agent(&ws->cnt[b][g], (unsigned)tot);
  // Everything another workgroup reads was stored at device scope (written through; such a store is complete once the
  // wave's store counter has drained), so every wave waits for its own stores, the barrier collects the waves, and the
  // ticket follows: no write-back or invalidation of the whole L2, which costs microseconds with a row per workgroup
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    s_last = atomicAdd(&ws->ticket[b][0], 1u) == (unsigned)(G - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // what follows reads the other workgroups' data at device scope

  // ---- the row's last workgroup
  int64_t* out_slot = out + pos_off + (size_t)b * out_stride;
  // every slot of the row's candidate lists is fetched together with the counts that say which of them are filled:
  // one trip to memory instead of two
  constexpr int PER = SAMP_MAX_CHUNKS * SAMP_CHUNK_CAP / 256;
  unsigned val[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int q = tid + u * 256;
    val[u] = (q / SAMP_CHUNK_CAP < G) ? ld_agent(&ws->cand[b][0][0] + q) : 0u;
  }
  if (w == 0) {
    const int c = lane < G ? (int)ld_agent(&ws->cnt[b][lane]) : 0;
    int ci = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(ci, o, FSTU_WAVE);
      if (lane >= o) ci += t;
    }
    if (lane <= G) s_off[lane] = ci - c;   // lane G: the total (its own count is 0)
    if (lane == 63) s_n = ci;
    const unsigned long long ov = __ballot(c > SAMP_CHUNK_CAP);
    if (lane == 0) s_over = ov != 0ull;
    best[(size_t)b * 64 + lane] = 0ull;
  }
  __syncthreads();
  if (s_over) {
    sample_row<bf16_t, false, 256>(sh, nullptr, row, out_slot, V, temperature, top_k, top_p, 1, seed, step, b + row0);
  } else {
    const int n = s_n;
    {
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int q = tid + u * 256, gq = q / SAMP_CHUNK_CAP, j = q % SAMP_CHUNK_CAP;
        if (gq < G && j < s_off[gq + 1] - s_off[gq]) {
          c_idx[s_off[gq] + j] = (unsigned short)(val[u] >> 16);
          c_key[s_off[gq] + j] = (unsigned short)(val[u] & 0xffffu);
        }
      }
    }
    __syncthreads();
    if (w == 0) {
      // maximum and its lowest index from the slots
      unsigned long long kb = slot;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long t = __shfl_xor(kb, o, FSTU_WAVE);
        kb = t > kb ? t : kb;
      }
      const float m = key_f32((unsigned)(kb >> 32));
      const int arg = (int)(0xffffffffu - (unsigned)(kb & 0xffffffffull));
      // the top_k-th largest key of the row is the top_k-th largest of the candidates
      unsigned thr = 0;
      if (n <= 128) {
        // the usual case: two keys per lane, held in registers (key 0 never counts: every trial value has a bit set)
        const unsigned k0 = lane < n ? (unsigned)c_key[lane] : 0u, k1 = lane + 64 < n ? (unsigned)c_key[lane + 64] : 0u;
#pragma unroll
        for (int bit = 15; bit >= 0; --bit) {
          const unsigned cnd = thr | (1u << bit);
          if (__popcll(__ballot(k0 >= cnd)) + __popcll(__ballot(k1 >= cnd)) >= top_k) thr = cnd;
        }
      } else {
        for (int bit = 15; bit >= 0; --bit) {
          const unsigned cnd = thr | (1u << bit);
          int c = 0;
          for (int i0 = 0; i0 < n; i0 += 64) {
            const int i = i0 + lane;
            c += __popcll(__ballot(i < n && (unsigned)c_key[i] >= cnd));
          }
          if (c >= top_k) thr = cnd;
        }
      }
      for (int i = lane; i < n; i += 64) {
        const unsigned k = c_key[i];
        c_e[i] = k >= thr ? expf(key16_f32(k) - m) : 0.f;
      }
      // ---- top-p over the survivors: kept set = {key > vb} U {key == vb with tie rank < tie_keep}
      unsigned vb = thr;
      long long tie_keep = -1;   // -1: keep every tied token
      if (top_p > 0.f && top_p < 1.f) {
        double e = 0.0;
        for (int i = lane; i < n; i += 64) e += (double)c_e[i];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) e += __shfl_xor(e, o, FSTU_WAVE);
        const double scale = 17592186044416.0 / e;   // 2^44 / Z1: fixed-point probabilities
        const unsigned long long target = (unsigned long long)((double)top_p * 17592186044416.0);
        for (int i = lane; i < n; i += 64) c_mass[i] = (unsigned long long)((double)c_e[i] * scale);
        // the largest key whose mass, together with everything above it, exceeds the target
        unsigned tbest = 0;
        bool any = false;
        for (int i0 = 0; i0 < n; i0 += 64) {
          const int i = i0 + lane;
          const bool ok = i < n && (unsigned)c_key[i] >= thr;
          const unsigned ki = ok ? (unsigned)c_key[i] : 0xffffffffu;
          unsigned long long S = 0ull;
          for (int j = 0; j < n; ++j)
            if ((unsigned)c_key[j] >= ki) S += c_mass[j];
          if (ok && S > target) { any = true; tbest = max(tbest, ki); }
        }
        if (__ballot(any) != 0ull) {
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) tbest = max(tbest, (unsigned)__shfl_xor((int)tbest, o, FSTU_WAVE));
          vb = tbest;
          unsigned long long above = 0ull;
          for (int i = lane; i < n; i += 64)
            if ((unsigned)c_key[i] > vb) above += c_mass[i];
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) above += __shfl_xor(above, o, FSTU_WAVE);
          unsigned long long pb = (unsigned long long)((double)expf(key16_f32(vb) - m) * scale);
          if (pb == 0ull) pb = 1ull;
          tie_keep = (long long)((target - above) / pb) + 1;
        }
      }
      // ---- draw: inverse CDF in index order over contiguous per-lane segments
      const int seg = (n + 63) / 64, i0 = min(n, lane * seg), i1 = min(n, i0 + seg);
      int tbase = 0;
      if (tie_keep >= 0) {
        int tc = 0;
        for (int i = i0; i < i1; ++i) tc += (unsigned)c_key[i] == vb;
        int ti = tc;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const int t = __shfl_up(ti, o, FSTU_WAVE);
          if (lane >= o) ti += t;
        }
        tbase = ti - tc;
      }
      double mysum = 0.0;
      {
        long long rank = tbase;
        for (int i = i0; i < i1; ++i) {
          const unsigned k = c_key[i];
          bool keep = k > vb;
          if (k == vb) { keep = (tie_keep < 0) || (rank < tie_keep); ++rank; }
          if (keep) mysum += (double)c_e[i];
        }
      }
      double si = mysum;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const double t = __shfl_up(si, o, FSTU_WAVE);
        if (lane >= o) si += t;
      }
      const double Z = __shfl(si, 63, FSTU_WAVE), mybase = si - mysum;
      // counter-based uniform (splitmix64 finaliser), 24 bits
      unsigned long long z = seed * 0x9E3779B97F4A7C15ull + (unsigned long long)step * 0xBF58476D1CE4E5B9ull +
                             (unsigned long long)(b + row0) * 0x94D049BB133111EBull + 0x2545F4914F6CDD1Dull;
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      z = z ^ (z >> 31);
      const double tgt = ((double)(z >> 40) / 16777216.0) * Z;
      int pick = -1;
      if (mysum > 0.0 && tgt >= mybase && tgt < mybase + mysum) {
        double acc = mybase;
        long long rank = tbase;
        int lastkept = -1;
        for (int i = i0; i < i1; ++i) {
          const unsigned k = c_key[i];
          bool keep = k > vb;
          if (k == vb) { keep = (tie_keep < 0) || (rank < tie_keep); ++rank; }
          if (keep) {
            acc += (double)c_e[i];
            lastkept = c_idx[i];
            if (acc > tgt) { pick = c_idx[i]; break; }
          }
        }
        if (pick < 0) pick = lastkept;
      }
      const unsigned long long who = __ballot(pick >= 0);
      if (who != 0ull) pick = __shfl(pick, __ffsll((long long)who) - 1, FSTU_WAVE);
      else pick = arg;   // rounding left the target past the last segment
      if (lane == 0) *out_slot = pick;
    }
  }
  // ---- leave the workspace as it was found
  if (tid < G) ws->cnt[b][tid] = 0u;
  if (tid == 0) {
    ws->ticket[b][0] = 0u;
    if (atomicAdd(&ws->done, 1u) == (unsigned)(nrows - 1)) {
      ws->done = 0u;
      if (dyn && advance) { dyn[0] = pos_off + 1; dyn[1] = step + 1; }
    }
  }
}

extern "C" int64_t fstu_sample_ws_bytes(void) { return (int64_t)sizeof(SampWs); }

bool fstu_sample_topk_ok(int B, int V, int top_k, int dtype) {
  return dtype == FSTU_BF16 && B >= 1 && B <= SAMP_MAX_ROWS && V >= 1024 && V <= SAMP_CHUNK * SAMP_MAX_CHUNKS && top_k >= 1 &&
         top_k <= 64;
}

int fstu_sample_topk_dyn(const void* logits, int64_t ldl, void* best_ws, void* samp_ws, int64_t* out, int64_t out_stride, int B,
                         int V, float temperature, int top_k, float top_p, uint64_t seed, int step, int row0, int* dyn,
                         int advance, void* stream) {
  FSTU_REQUIRE(logits && best_ws && samp_ws && out, FSTU_ENULL, "fstu_sample_topk: null pointer");
  FSTU_REQUIRE(fstu_sample_topk_ok(B, V, top_k, FSTU_BF16), FSTU_ESHAPE,
               "fstu_sample_topk: needs 1 <= B <= %d, 1024 <= V <= %d, 1 <= top_k <= 64 (B=%d V=%d top_k=%d)", SAMP_MAX_ROWS,
               SAMP_CHUNK * SAMP_MAX_CHUNKS, B, V, top_k);
  FSTU_REQUIRE(temperature > 0.f && ldl >= V && out_stride >= 1, FSTU_EARG, "fstu_sample_topk: bad temperature / ldl / out_stride");
  FSTU_REQUIRE(fstu_aligned(best_ws, 8) && fstu_aligned(samp_ws, 8) && fstu_aligned(logits, 2), FSTU_EALIGN,
               "fstu_sample_topk: workspaces must be 8-byte aligned");
  const dim3 grid((V + SAMP_CHUNK - 1) / SAMP_CHUNK, B);
  hipLaunchKernelGGL(sample_topk_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)logits, ldl,
                     (unsigned long long*)best_ws, (SampWs*)samp_ws, out, out_stride, V, temperature, top_k, top_p, seed, step, row0,
                     dyn, advance);
  FSTU_CHECK_LAUNCH("fstu_sample_topk");
  return FSTU_OK;
}

extern "C" int fstu_sample_topk(const void* logits, int64_t ldl, void* best_ws, void* samp_ws, int64_t* out, int64_t out_stride,
                                int B, int V, float temperature, int top_k, float top_p, uint64_t seed, int step, void* stream) {
  return fstu_sample_topk_dyn(logits, ldl, best_ws, samp_ws, out, out_stride, B, V, temperature, top_k, top_p, seed, step, 0, nullptr,
                              0, stream);
}

__global__ void advance_dyn_kernel(int* dyn) {
  if (threadIdx.x == 0) { dyn[0] += 1; dyn[1] += 1; }
}

int fstu_advance_dyn(int* dyn, void* stream) {
  hipLaunchKernelGGL(advance_dyn_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, dyn);
  FSTU_CHECK_LAUNCH("fstu_advance_dyn");
  return FSTU_OK;
}

extern "C" int fstu_sample(const void* logits, int64_t* out, int64_t out_stride, int B, int V, float temperature,
                           int top_k, float top_p, int do_sample, uint64_t seed, int step, int dtype,
                           void* stream) {
  return fstu_sample_dyn(logits, out, out_stride, B, V, temperature, top_k, top_p, do_sample, seed, step, 0, nullptr, dtype,
                         stream);
}

int fstu_sample_dyn(const void* logits, int64_t* out, int64_t out_stride, int B, int V, float temperature, int top_k,
                    float top_p, int do_sample, uint64_t seed, int step, int row0, const int* dyn, int dtype, void* stream) {
  FSTU_REQUIRE(logits && out, FSTU_ENULL, "fstu_sample: null pointer");
  FSTU_REQUIRE(B >= 0 && V > 0, FSTU_ESHAPE, "fstu_sample: bad shape B=%d V=%d", B, V);
  FSTU_REQUIRE(temperature > 0.f, FSTU_EARG, "fstu_sample: temperature must be > 0");
  FSTU_REQUIRE(out_stride >= 1, FSTU_EARG, "fstu_sample: out_stride < 1");
  if (B == 0) return FSTU_OK;
  if (dtype == FSTU_BF16 && do_sample && V <= 65536) {
    const size_t shm = ((size_t)V * 2 + 15) & ~(size_t)15;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(sample_kernel<bf16_t, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    FSTU_REQUIRE(e == hipSuccess, (int)e, "fstu_sample: %d bytes of dynamic LDS refused", 128 * 1024);
    hipLaunchKernelGGL((sample_kernel<bf16_t, true>), dim3(B), dim3(FSTU_SAMPLE_THREADS), shm, (hipStream_t)stream,
                       (const bf16_t*)logits, out, out_stride, V, temperature, top_k, top_p, do_sample, seed, step, row0, dyn);
    FSTU_CHECK_LAUNCH("fstu_sample");
    return FSTU_OK;
  }
  FSTU_DISPATCH_DTYPE(dtype, "fstu_sample",
                      hipLaunchKernelGGL((sample_kernel<T, false>), dim3(B), dim3(FSTU_SAMPLE_THREADS), 0, (hipStream_t)stream,
                                         (const T*)logits, out, out_stride, V, temperature, top_k, top_p, do_sample,
                                         seed, step, row0, dyn));
  FSTU_CHECK_LAUNCH("fstu_sample");
  return FSTU_OK;
}
