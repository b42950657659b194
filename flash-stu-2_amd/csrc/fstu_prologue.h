// Norm prologue of the decode GEMV kernels: the residual update and the RMSNorm of ALL rows, recomputed by every
// workgroup in front of its own slice of a projection, so that the separate add+norm launch between two projections
// disappears (reference wiring: flash_stu/layers/stu_layer.py:78-97, attention_layer.py:50-66).
//
//   x' = T(x + delta)                         delta: bf16 rows, or the fixed-order sum of up to NS fp32 split-K slices
//                                             rounded to bf16 first (what fstu_add_rmsnorm does with delta_mode 1)
//   h  = T((x' * rsqrt(mean(x'^2) + eps)) * w)
//
// Thread q of the workgroup owns chunk q (8 channels) of the (rows x d/8) grid from load to store; a row is a whole
// number of 32-lane groups (d % 256 == 0), so the row statistics need one 32-lane reduction and d/256 partials per
// row in LDS.  The three phases are separate calls so that a kernel can put its own weight loads between them.
#pragma once
#include "fstu_common.h"

typedef __amdgpu_buffer_rsrc_t fstu_rsrc_t;
typedef unsigned int fstu_u32x4_t __attribute__((ext_vector_type(4)));
#define FSTU_BUF_OOB 0xfffffff0u

// Raw buffer loads: a lane whose byte offset lies beyond the descriptor's range reads zeros without a branch, so the
// load stays in straight-line code and the compiler's load-counter bookkeeping stays exact.
__device__ __forceinline__ fstu_rsrc_t fstu_make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, p ? (unsigned)bytes : 0u, 0x00020000);
}
__device__ __forceinline__ uint4 fstu_buf_load16(fstu_rsrc_t rs, unsigned off) {
  fstu_u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// sum over each aligned group of 32 lanes, returned in every lane of the group
__device__ __forceinline__ float fstu_half_wave_sum(float v) {
  v += fstu_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  v += fstu_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  v += fstu_dpp<0x141>(v);   // row_half_mirror
  v += fstu_dpp<0x140>(v);   // row_mirror
  return v + fstu_swz16(v);
}

template <int NT, int NXC, int NS>
struct NormPrologue {
  static constexpr int NSV = NS > 0 ? NXC * NS * 2 : 1;
  static constexpr int NPART = NXC * NT / 32;   // floats of LDS for the partial sums
  uint4 xv[NXC], nv[NXC], dv[NS > 0 ? 1 : NXC];
  uint4 sv[NSV];
  int rowj[NXC];

  // the caller picks the smallest NXC with rows * d/8 <= NXC * NT: every j below then has chunks to do, and the code
  // is one straight line (lanes beyond the last chunk read zeros and store nothing)
  static __host__ __device__ bool supported(int rows, int d) {
    return d % 256 == 0 && rows >= 1 && (long long)rows * (d / 8) <= (long long)NXC * NT;
  }

  // phase 1: every load of the prologue, in straight-line code.  x_in and delta point at the first of the `rows` rows;
  // when these are a few rows of taller slices, slice_chunks is the distance between two slices in 8-channel chunks.
  __device__ __forceinline__ void issue(const bf16_t* x_in, const void* delta, int nslices, const bf16_t* norm_w, int rows,
                                        int d, int slice_chunks = 0) {
    const int nchunk = d >> 3, total = rows * nchunk;
    const int sstride = slice_chunks > 0 ? slice_chunks : total;
    const fstu_rsrc_t rx = fstu_make_rsrc(x_in, (size_t)total * 16);
    const fstu_rsrc_t rd = fstu_make_rsrc(
        delta, NS > 0 ? (nslices > 0 ? ((size_t)(nslices - 1) * sstride + total) * 32 : 0) : (size_t)total * 16);
    const fstu_rsrc_t rn = fstu_make_rsrc(norm_w, (size_t)d * 2);
    const float inv_nc = 1.0f / (float)nchunk;
#pragma unroll
    for (int j = 0; j < NXC; ++j) {
      const int q = threadIdx.x + j * NT;
      rowj[j] = (int)(((float)q + 0.5f) * inv_nc);
      xv[j] = fstu_buf_load16(rx, (unsigned)q * 16u);     // beyond the last chunk: zeros
      if (NS > 0) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          // slices beyond nslices lie beyond the descriptor's range: zeros
          const unsigned off = q < total ? ((unsigned)s * (unsigned)sstride + (unsigned)q) * 32u : FSTU_BUF_OOB;
          sv[(j * NS + s) * 2] = fstu_buf_load16(rd, off);
          sv[(j * NS + s) * 2 + 1] = fstu_buf_load16(rd, q < total ? off + 16u : FSTU_BUF_OOB);
        }
      } else {
        dv[j] = fstu_buf_load16(rd, (unsigned)q * 16u);   // no delta: zeros
      }
      nv[j] = fstu_buf_load16(rn, (unsigned)(q - rowj[j] * nchunk) * 16u);
    }
  }

  // phase 2: x' into xv (and to x_out when given), the 32-lane partial sums of x'^2 into ss_part[NPART]
  __device__ __forceinline__ void reduce(float* ss_part, bf16_t* x_out, int rows, int d) {
    const int nchunk = d >> 3, total = rows * nchunk;
#pragma unroll
    for (int j = 0; j < NXC; ++j) {
      const int q = threadIdx.x + j * NT;
      unsigned xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w};
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float dlo, dhi;
        if (NS > 0) {
          float tlo = 0.f, thi = 0.f;
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            const uint4 p = sv[(j * NS + s) * 2 + (i >> 1)];
            tlo += __uint_as_float((i & 1) ? p.z : p.x);
            thi += __uint_as_float((i & 1) ? p.w : p.y);
          }
          const unsigned dp = pack2_bf16(tlo, thi);
          dlo = __uint_as_float(dp << 16);
          dhi = __uint_as_float(dp & 0xffff0000u);
        } else {
          const unsigned dw = i == 0 ? dv[j].x : (i == 1 ? dv[j].y : (i == 2 ? dv[j].z : dv[j].w));
          dlo = __uint_as_float(dw << 16);
          dhi = __uint_as_float(dw & 0xffff0000u);
        }
        xw[i] = pack2_bf16(__uint_as_float(xw[i] << 16) + dlo, __uint_as_float(xw[i] & 0xffff0000u) + dhi);
        const float lo = __uint_as_float(xw[i] << 16), hi = __uint_as_float(xw[i] & 0xffff0000u);
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
      }
      xv[j] = make_uint4(xw[0], xw[1], xw[2], xw[3]);
      ss = fstu_half_wave_sum(ss);
      if ((threadIdx.x & 31) == 0) ss_part[q >> 5] = ss;
      if (x_out && q < total) *(uint4*)(x_out + (size_t)q * 8) = xv[j];
    }
  }

  // Makes the loaded values opaque at this point of the program: arithmetic of reduce() that depends on a single load
  // (the first term of a slice sum) can then not be hoisted to the loads, where its wait would stall whatever the
  // caller issues between issue() and reduce().
  __device__ __forceinline__ void pin_loads() {
    if (NS > 0) {
#pragma unroll
      for (int k = 0; k < NSV; ++k) asm volatile("" : "+v"(sv[k].x), "+v"(sv[k].y), "+v"(sv[k].z), "+v"(sv[k].w));
    }
  }

  // the norm weights have arrived (keeps later loads of the caller from having to be waited for with them)
  __device__ __forceinline__ void pin_weights() {
#pragma unroll
    for (int j = 0; j < NXC; ++j)
      asm volatile("" ::"v"(nv[j].x), "v"(nv[j].y), "v"(nv[j].z), "v"(nv[j].w));
  }

  // phase 3 (after a __syncthreads()): h rows into LDS, row stride ld elements
  __device__ __forceinline__ void scale(const float* ss_part, bf16_t* hs, int ld, int rows, int d, float eps) {
    const int nchunk = d >> 3, total = rows * nchunk, gpr = nchunk >> 5;
    const float inv_d = 1.0f / (float)d;
#pragma unroll
    for (int j = 0; j < NXC; ++j) {
      const int q = threadIdx.x + j * NT;
      if (q < total) {
        float ss = 0.f;
        const float* sp = ss_part + rowj[j] * gpr;
        for (int i = 0; i < gpr; ++i) ss += sp[i];
        const float rstd = rsqrtf(ss * inv_d + eps);
        unsigned vw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, ww[4] = {nv[j].x, nv[j].y, nv[j].z, nv[j].w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          vw[i] = pack2_bf16((__uint_as_float(vw[i] << 16) * rstd) * __uint_as_float(ww[i] << 16),
                             (__uint_as_float(vw[i] & 0xffff0000u) * rstd) * __uint_as_float(ww[i] & 0xffff0000u));
        *(uint4*)(hs + (size_t)rowj[j] * ld + (size_t)(q - rowj[j] * nchunk) * 8) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
      }
    }
  }
};
