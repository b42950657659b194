// Shared device/host helpers for the gfx950 kernels of libflashstu_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/flashstu_hip.h"

#define FSTU_WAVE 64

// ---------------------------------------------------------------- errors
void fstu_set_error(const char* fmt, ...);

#define FSTU_REQUIRE(cond, code, ...)                 \
  do {                                                \
    if (!(cond)) {                                    \
      fstu_set_error(__VA_ARGS__);                    \
      return (code);                                  \
    }                                                 \
  } while (0)

#define FSTU_CHECK_LAUNCH(name)                                           \
  do {                                                                    \
    hipError_t e__ = hipGetLastError();                                   \
    if (e__ != hipSuccess) {                                              \
      fstu_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
      return (int)e__;                                                    \
    }                                                                     \
  } while (0)

// ---- library-internal launchers used by the decode-step driver.  `dyn`, when not null, is a device int[2]
// {position, sampling step} read by the kernels instead of the host-side values, so that a captured graph of one
// step can be replayed for every position.
extern "C" int fstu_stu_lds_state_ring_from_hist(const void* hist, const float* a, float* state, void* ring, int R, int B,
                                                 int S, int d, int t_last, int cap, int dtype, void* stream);
int fstu_embed_strided(const int64_t* ids, int64_t id_stride, const void* table, void* out, int rows, int d, int vocab,
                       int dtype, void* stream, const int* dyn);
int fstu_stu_step_lds_dyn(float* state, const void* xp, int ldxp, const float* a, const float* ce, void* y, int ldy,
                          int B, int S, int d, int t, const int* dyn, int dtype, void* stream);
int fstu_swa_decode_impl(const void* qkv, void* kring, void* vring, void* out, const float* slopes, int B, int H, int hd,
                         int cap, int pos, int window, float softcap, int append, const int* dyn, int dtype, void* stream);
int fstu_head_argmax_dyn(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                         float temperature, void* best_ws, int64_t* tok_out, int64_t tok_stride, int* dyn, int advance,
                         int dtype, void* stream);
int fstu_argmax_finish_launch(void* best_ws, int64_t* tok_out, int64_t tok_stride, int rows, int* dyn, int advance, void* stream);
bool fstu_finish_embed_supported(int rows, int d, const void* table, const void* x, const void* w, const void* h);
int fstu_finish_embed_rmsnorm(void* best_ws, int64_t* tok_out, int64_t tok_stride, const void* table, void* x, const void* w,
                              void* h, int* dyn, int rows, int d, int vocab, float eps, void* stream);
bool fstu_head_argmax_fused_pick(const void* x, int ldx, const void* W, int K, int dtype);
int fstu_embed_rmsnorm(const int64_t* ids, int64_t id_stride, const void* table, void* x, const void* w, void* h, int rows,
                       int d, int vocab, float eps, int dtype, void* stream, const int* dyn);
int fstu_sample_dyn(const void* logits, int64_t* out, int64_t out_stride, int B, int V, float temperature, int top_k,
                    float top_p, int do_sample, uint64_t seed, int step, int row0, const int* dyn, int dtype, void* stream);
int fstu_advance_dyn(int* dyn, void* stream);
bool fstu_linear_rows32_ok(const void* x, int ldx, const void* W, int K, int dtype);
int fstu_linear_rows32(const void* x, int ldx, const void* W, void* y, int ldy, int rows, int N, int K, float temperature,
                       void* best_ws /*NULL: plain projection; else the head's packed maxima, rows*64 words*/, void* stream);
bool fstu_sample_topk_ok(int B, int V, int top_k, int dtype);
int fstu_sample_topk_dyn(const void* logits, int64_t ldl, void* best_ws, void* samp_ws, int64_t* out, int64_t out_stride, int B,
                         int V, float temperature, int top_k, float top_p, uint64_t seed, int step, int row0, int* dyn,
                         int advance, void* stream);
int fstu_stu_step_lds_pair_dyn(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co, void* ring,
                               const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int t, const int* dyn,
                               const int* pos_dyn, int dtype, void* stream,
                               const void* res = nullptr /*y = T(res + T(output)), rows of stride ldy*/,
                               float* ocache = nullptr /*(B,d): the odd-lag sum handed from step to step*/);
int fstu_stu_inproj_step_dyn(const void* h, int ldh, const void* Mt, float* state, const float* a, const float* ce,
                             const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, void* xp_out, int B,
                             int S, int d, int K, int t, const int* dyn, const int* pos_dyn, void* stream);
int fstu_stu_res_inproj_step_dyn(const void* x_in, const float* slices, int nslices, void* x_out, const void* norm_w, float eps,
                                 const void* Mt, float* state, const float* a, const float* ce, const float* co, void* ring,
                                 const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int K, int t,
                                 const int* dyn, const int* pos_dyn, void* stream);
static inline bool fstu_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
// the optional exact head of the distilled filter: ring, taps and their count go together; count a power of two in 8..1024
static inline bool fstu_fir_ok(const void* ring, const float* fir, int taps) {
  if (!ring && !fir && taps == 0) return true;
  return ring && fir && taps >= 8 && taps <= 1024 && (taps & (taps - 1)) == 0 && fstu_aligned(ring, 16) && fstu_aligned(fir, 16);
}

// ---------------------------------------------------------------- dtypes
typedef unsigned short bf16_t;  // raw bf16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((unsigned)v) << 16); }

// round-to-nearest-even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32, two values per instruction).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }
// (lo, hi) -> two bf16 in one word, lo in the low half
__device__ __forceinline__ unsigned pack2_bf16(float lo, float hi) {
  typedef float fstu_f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 fstu_bf16x2 __attribute__((ext_vector_type(2)));
  fstu_f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, fstu_bf16x2));
}

template <typename T> struct DT;
template <> struct DT<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
};
template <> struct DT<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  static __device__ __forceinline__ float rnd(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

// ---------------------------------------------------------------- wave ops
// All-lane reductions of a 64-wide wave, every lane active: four DPP steps inside a row of 16 lanes, one swizzle
// across the two rows of a half, two lane reads across the halves (no LDS round trips).
template <int CTRL>
__device__ __forceinline__ float fstu_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float fstu_swz16(float v) {   // value of lane ^ 16
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += fstu_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  v += fstu_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  v += fstu_dpp<0x141>(v);   // row_half_mirror
  v += fstu_dpp<0x140>(v);   // row_mirror
  v += fstu_swz16(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) +
         __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, fstu_dpp<0xB1>(v));
  v = fmaxf(v, fstu_dpp<0x4E>(v));
  v = fmaxf(v, fstu_dpp<0x141>(v));
  v = fmaxf(v, fstu_dpp<0x140>(v));
  v = fmaxf(v, fstu_swz16(v));
  return fmaxf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)),
               __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)));
}

// tanh-approximated GELU as torch evaluates it in fp32
__device__ __forceinline__ float gelu_tanh_f32(float x) {
  const float kBeta = 0.7978845608028654f;  // sqrt(2/pi)
  const float kKappa = 0.044715f;
  float inner = kBeta * (x + kKappa * x * x * x);
  return 0.5f * x * (1.0f + tanhf(inner));
}

#define FSTU_DISPATCH_DTYPE(dtype, NAME, ...)                      \
  do {                                                             \
    if ((dtype) == FSTU_F32) {                                     \
      typedef float T;                                             \
      __VA_ARGS__;                                                 \
    } else if ((dtype) == FSTU_BF16) {                             \
      typedef bf16_t T;                                            \
      __VA_ARGS__;                                                 \
    } else {                                                       \
      fstu_set_error("%s: unknown dtype %d", NAME, (int)(dtype));  \
      return FSTU_EDTYPE;                                          \
    }                                                              \
  } while (0)
