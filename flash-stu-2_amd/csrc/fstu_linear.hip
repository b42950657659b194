// Skinny linear layers for decode: up to 16 activation rows against an (N,K)
// weight that is streamed from HBM exactly once.
//
// bf16 path: one wave owns a 16-feature row tile and a K range.  The weight
// tile is the MFMA A operand (16 features x 32 k), the activations the B
// operand (32 k x 16 batch rows, rows >= `rows` are zero), accumulated with
// v_mfma_f32_16x16x32_bf16.  Within one 64-wide k step lane (r,g) reads the 32
// contiguous bytes W[r, k+16g .. k+16g+15], so the four lanes of a row cover a
// full 128-byte line; the two MFMAs of the step take the low and high 8
// elements and the activation operand is permuted identically (a dot product
// does not care about the order of k).
// Waves of a workgroup that share a row tile but own different K ranges are
// reduced through LDS in a fixed order, so results are deterministic.
//
// Other dtypes/shapes: a vector-ALU kernel, one wave per output feature.
#include "fstu_common.h"
#include <mutex>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

enum { LIN_PLAIN = 0, LIN_GLU = 1, LIN_PARTIAL = 2, LIN_ARGMAX = 3 };

struct LinArgs {
  const void* x;
  int ldx;
  const void* W;   // plain weight or gate weight
  const void* W2;  // up weight (GLU)
  void* y;         // T output (plain/GLU) or fp32 partial slices
  int ldy;
  int rows, N, K;
  int kw;          // k range per wave
  unsigned long long* best;  // LIN_ARGMAX: per-row packed (value key, ~index) maxima, zero on entry
  float temperature;         // LIN_ARGMAX: logits are divided by it before comparison
};

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }

// The arguments are passed one by one (not as a struct) so that the command processor can preload them into SGPRs.
// NB = 2: rows 16..31 are a second B tile of the same weight fragments, so 17..32 rows read every weight once.
template <int KSW, int MODE, int NB = 1>
__global__ void __launch_bounds__(256)
linear_mfma_bf16_kernel(const void* x, const void* W, const void* W2, void* y, unsigned long long* best, int ldx, int ldy,
                        int rows, int N, int K, int kw, float temperature) {
  static_assert(NB == 1 || MODE == LIN_PLAIN || MODE == LIN_ARGMAX, "two row tiles: plain and head launches only");
  const LinArgs a{x, ldx, W, W2, y, ldy, rows, N, K, kw, best, temperature};
  constexpr int RT = 4 / KSW;
  constexpr int U = 4;  // k steps (of 64) whose loads are issued back to back
  constexpr int NACC = (MODE == LIN_GLU) ? 2 : NB;   // accumulators per lane: gate + up, or one per row tile
  __shared__ float red[(KSW > 1) ? 4 * 64 * 4 * NACC : 1];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int rt = w / KSW, ks = w % KSW;
  const int tile = blockIdx.x * RT + rt;
  const int ntiles = (a.N + 15) >> 4;
  const bool tile_ok = tile < ntiles;
  const int r = lane & 15, g = lane >> 4;
  const int n = min(tile * 16 + r, a.N - 1);
  const int k0 = (blockIdx.y * KSW + ks) * a.kw + g * 16;
  const bf16_t* wp = (const bf16_t*)a.W + (size_t)max(n, 0) * a.K + k0;
  const bf16_t* wp2 = (MODE == LIN_GLU) ? (const bf16_t*)a.W2 + (size_t)max(n, 0) * a.K + k0 : nullptr;
  bool xrow[NB];
  const bf16_t* xp[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    xrow[j] = 16 * j + r < a.rows;
    xp[j] = (const bf16_t*)a.x + (size_t)(xrow[j] ? 16 * j + r : 0) * a.ldx + k0;
  }
  floatx4_t acc[NACC];
#pragma unroll
  for (int j = 0; j < NACC; ++j) acc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  const int iters = a.kw >> 6;
  if (tile_ok) {
    for (int i0 = 0; i0 < iters; i0 += U) {
      uint4 wa[U][2], wb[U][2], xa[NB][U][2];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + u < iters) {
          const uint4* p = (const uint4*)(wp + (size_t)(i0 + u) * 64);
          wa[u][0] = p[0];
          wa[u][1] = p[1];
          if (MODE == LIN_GLU) {
            const uint4* p2 = (const uint4*)(wp2 + (size_t)(i0 + u) * 64);
            wb[u][0] = p2[0];
            wb[u][1] = p2[1];
          }
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            if (xrow[j]) {
              const uint4* q = (const uint4*)(xp[j] + (size_t)(i0 + u) * 64);
              xa[j][u][0] = q[0];
              xa[j][u][1] = q[1];
            } else {
              xa[j][u][0] = make_uint4(0, 0, 0, 0);
              xa[j][u][1] = make_uint4(0, 0, 0, 0);
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + u < iters) {
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[u][0]), as_bf16x8(xa[j][u][0]), acc[j], 0, 0, 0);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wa[u][1]), as_bf16x8(xa[j][u][1]), acc[j], 0, 0, 0);
          }
          if (MODE == LIN_GLU) {
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb[u][0]), as_bf16x8(xa[0][u][0]), acc[1], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wb[u][1]), as_bf16x8(xa[0][u][1]), acc[1], 0, 0, 0);
          }
        }
      }
    }
  }
  if (KSW > 1) {
    float* mine = red + (size_t)(w * 64 + lane) * 4;
    constexpr int OFF = 4 * 64 * 4;
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[j * OFF + i] = acc[j][i];
    __syncthreads();
    if (ks != 0) return;
#pragma unroll
    for (int s = 1; s < KSW; ++s) {
      const float* o = red + (size_t)((w + s) * 64 + lane) * 4;
#pragma unroll
      for (int j = 0; j < NACC; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] += o[j * OFF + i];
    }
  }
  if (MODE == LIN_ARGMAX) {
    // per batch row: best (value, lowest index) over this wave's 16 features, then one 64-bit atomic max
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int b = 16 * j + r;
      unsigned long long key = 0ull;
      if (tile_ok && b < a.rows) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int f = tile * 16 + g * 4 + i;
          if (f < a.N) {
            float l = DT<bf16_t>::rnd(acc[j][i]);
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
      if (tile_ok && g == 0 && b < a.rows && key != 0ull) atomicMax(a.best + (size_t)b * 64 + (tile & 63), key);  // 64 slots per row spread the contention
    }
  }
  if (!tile_ok) return;
  // D layout: lane holds features 4*(lane/16)+i, batch row lane%16 (of its row tile)
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int b = 16 * j + r;
    if (b >= a.rows) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int f = tile * 16 + g * 4 + i;
      if (f >= a.N) continue;
      if (MODE == LIN_PLAIN || MODE == LIN_ARGMAX) {
        ((bf16_t*)a.y)[(size_t)b * a.ldy + f] = f32_to_bf16(acc[j][i]);
      } else if (MODE == LIN_GLU) {
        float ge = DT<bf16_t>::rnd(gelu_tanh_f32(DT<bf16_t>::rnd(acc[0][i])));
        ((bf16_t*)a.y)[(size_t)b * a.ldy + f] = f32_to_bf16(ge * DT<bf16_t>::rnd(acc[1][i]));
      } else {
        ((float*)a.y)[((size_t)blockIdx.y * a.rows + b) * a.N + f] = acc[j][i];
      }
    }
  }
}

// Vector-ALU kernel: one wave per output feature (and K split), lanes stride
// over k.  Any dtype, any K.
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
linear_valu_kernel(LinArgs a) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int n = blockIdx.x * 4 + w;
  if (n >= a.N) return;
  const int k0 = blockIdx.y * a.kw, k1 = min(a.K, k0 + a.kw);
  const T* wr = (const T*)a.W + (size_t)n * a.K;
  const T* wr2 = (MODE == LIN_GLU) ? (const T*)a.W2 + (size_t)n * a.K : nullptr;
  const T* x = (const T*)a.x;
  float acc[FSTU_MAX_DECODE_ROWS], acc2[FSTU_MAX_DECODE_ROWS];
#pragma unroll
  for (int b = 0; b < FSTU_MAX_DECODE_ROWS; ++b) { acc[b] = 0.f; acc2[b] = 0.f; }
  for (int k = k0 + lane; k < k1; k += 64) {
    float wv = DT<T>::ld(wr + k);
    float wv2 = (MODE == LIN_GLU) ? DT<T>::ld(wr2 + k) : 0.f;
#pragma unroll
    for (int b = 0; b < FSTU_MAX_DECODE_ROWS; ++b) {
      if (b < a.rows) {
        float xv = DT<T>::ld(x + (size_t)b * a.ldx + k);
        acc[b] = fmaf(wv, xv, acc[b]);
        if (MODE == LIN_GLU) acc2[b] = fmaf(wv2, xv, acc2[b]);
      }
    }
  }
#pragma unroll
  for (int b = 0; b < FSTU_MAX_DECODE_ROWS; ++b) {
    if (b < a.rows) {
      float s = wave_sum(acc[b]);
      float s2 = (MODE == LIN_GLU) ? wave_sum(acc2[b]) : 0.f;
      if (lane == 0) {
        if (MODE == LIN_PLAIN) {
          DT<T>::st((T*)a.y + (size_t)b * a.ldy + n, s);
        } else if (MODE == LIN_GLU) {
          float ge = DT<T>::rnd(gelu_tanh_f32(DT<T>::rnd(s)));
          DT<T>::st((T*)a.y + (size_t)b * a.ldy + n, ge * DT<T>::rnd(s2));
        } else {
          ((float*)a.y)[((size_t)blockIdx.y * a.rows + b) * a.N + n] = s;
        }
      }
    }
  }
}

static int check_common(const char* name, const void* x, const void* W, const void* y, int ldx, int rows, int N, int K) {
  FSTU_REQUIRE(x && W && y, FSTU_ENULL, "%s: null pointer", name);
  FSTU_REQUIRE(rows >= 1 && rows <= FSTU_MAX_DECODE_ROWS, FSTU_ESHAPE, "%s: rows=%d outside 1..%d", name, rows,
               FSTU_MAX_DECODE_ROWS);
  FSTU_REQUIRE(N >= 1 && K >= 1, FSTU_ESHAPE, "%s: N=%d K=%d", name, N, K);
  FSTU_REQUIRE(ldx >= K, FSTU_ESHAPE, "%s: ldx=%d < K=%d", name, ldx, K);
  return FSTU_OK;
}

static bool mfma_ok(const void* x, int ldx, const void* W, const void* W2, int K, int ksplit) {
  return K % (64 * ksplit) == 0 && ldx % 8 == 0 && fstu_aligned(x, 16) && fstu_aligned(W, 16) &&
         (W2 == nullptr || fstu_aligned(W2, 16));
}

// in-workgroup K split: use the deepest split that keeps >= 128 k per wave
static int pick_ksw(int N, int kper) {
  int tiles = (N + 15) / 16;
  if (kper % 256 == 0 && kper >= 512 && tiles < 4096) return 4;
  if (kper % 128 == 0 && kper >= 256 && tiles < 8192) return 2;
  return 1;
}

template <int MODE, int NB = 1>
static int launch_mfma(LinArgs a, int ksplit, hipStream_t s) {
  int kper = a.K / ksplit;
  int ksw = pick_ksw(a.N, kper);
  a.kw = kper / ksw;
  int tiles = (a.N + 15) / 16;
  int rt = 4 / ksw;
  dim3 grid((tiles + rt - 1) / rt, ksplit);
  if (ksw == 4) hipLaunchKernelGGL((linear_mfma_bf16_kernel<4, MODE, NB>), grid, dim3(256), 0, s, a.x, a.W, a.W2, a.y, a.best, a.ldx, a.ldy, a.rows, a.N, a.K, a.kw, a.temperature);
  else if (ksw == 2) hipLaunchKernelGGL((linear_mfma_bf16_kernel<2, MODE, NB>), grid, dim3(256), 0, s, a.x, a.W, a.W2, a.y, a.best, a.ldx, a.ldy, a.rows, a.N, a.K, a.kw, a.temperature);
  else hipLaunchKernelGGL((linear_mfma_bf16_kernel<1, MODE, NB>), grid, dim3(256), 0, s, a.x, a.W, a.W2, a.y, a.best, a.ldx, a.ldy, a.rows, a.N, a.K, a.kw, a.temperature);
  return 0;
}

// 17..32 rows (bf16, K % 64 == 0, 16-byte aligned rows): the plain projection and the head with its packed maxima,
// every weight read once.  Used by the one-call step for batches beyond FSTU_MAX_DECODE_ROWS.
bool fstu_linear_rows32_ok(const void* x, int ldx, const void* W, int K, int dtype) {
  return dtype == FSTU_BF16 && mfma_ok(x, ldx, W, nullptr, K, 1);
}

int fstu_linear_rows32(const void* x, int ldx, const void* W, void* y, int ldy, int rows, int N, int K, float temperature,
                       void* best_ws, void* stream) {
  FSTU_REQUIRE(x && W && y, FSTU_ENULL, "fstu_linear_rows32: null pointer");
  FSTU_REQUIRE(rows > FSTU_MAX_DECODE_ROWS && rows <= 2 * FSTU_MAX_DECODE_ROWS && N >= 1 && ldx >= K && ldy >= N, FSTU_ESHAPE,
               "fstu_linear_rows32: rows=%d N=%d K=%d ldx=%d ldy=%d", rows, N, K, ldx, ldy);
  FSTU_REQUIRE(mfma_ok(x, ldx, W, nullptr, K, 1), FSTU_ESHAPE, "fstu_linear_rows32: needs K %% 64 == 0 and 16-byte aligned rows");
  LinArgs a{x, ldx, W, nullptr, y, ldy, rows, N, K, K, (unsigned long long*)best_ws, temperature};
  if (best_ws) launch_mfma<LIN_ARGMAX, 2>(a, 1, (hipStream_t)stream);
  else launch_mfma<LIN_PLAIN, 2>(a, 1, (hipStream_t)stream);
  FSTU_CHECK_LAUNCH("fstu_linear_rows32");
  return FSTU_OK;
}

template <typename T, int MODE>
static void launch_valu(LinArgs a, int ksplit, hipStream_t s) {
  a.kw = (a.K + ksplit - 1) / ksplit;
  dim3 grid((a.N + 3) / 4, ksplit);
  hipLaunchKernelGGL((linear_valu_kernel<T, MODE>), grid, dim3(256), 0, s, a);
}

extern "C" int fstu_linear_decode(const void* x, int ldx, const void* W, void* y, int ldy, int rows, int N, int K,
                                  int dtype, void* stream) {
  int rc = check_common("fstu_linear_decode", x, W, y, ldx, rows, N, K);
  if (rc) return rc;
  FSTU_REQUIRE(ldy >= N, FSTU_ESHAPE, "fstu_linear_decode: ldy=%d < N=%d", ldy, N);
  LinArgs a{x, ldx, W, nullptr, y, ldy, rows, N, K, K, nullptr, 1.0f};
  if (dtype == FSTU_BF16) {
    if (mfma_ok(x, ldx, W, nullptr, K, 1)) launch_mfma<LIN_PLAIN>(a, 1, (hipStream_t)stream);
    else launch_valu<bf16_t, LIN_PLAIN>(a, 1, (hipStream_t)stream);
  } else if (dtype == FSTU_F32) {
    launch_valu<float, LIN_PLAIN>(a, 1, (hipStream_t)stream);
  } else {
    fstu_set_error("fstu_linear_decode: unknown dtype %d", dtype);
    return FSTU_EDTYPE;
  }
  FSTU_CHECK_LAUNCH("fstu_linear_decode");
  return FSTU_OK;
}

extern "C" int fstu_glu_decode(const void* x, int ldx, const void* Wg, const void* Wu, void* act, int ldact, int rows,
                               int I, int K, int dtype, void* stream) {
  int rc = check_common("fstu_glu_decode", x, Wg, act, ldx, rows, I, K);
  if (rc) return rc;
  FSTU_REQUIRE(Wu, FSTU_ENULL, "fstu_glu_decode: Wu is null");
  FSTU_REQUIRE(ldact >= I, FSTU_ESHAPE, "fstu_glu_decode: ldact=%d < I=%d", ldact, I);
  LinArgs a{x, ldx, Wg, Wu, act, ldact, rows, I, K, K, nullptr, 1.0f};
  if (dtype == FSTU_BF16) {
    if (mfma_ok(x, ldx, Wg, Wu, K, 1)) launch_mfma<LIN_GLU>(a, 1, (hipStream_t)stream);
    else launch_valu<bf16_t, LIN_GLU>(a, 1, (hipStream_t)stream);
  } else if (dtype == FSTU_F32) {
    launch_valu<float, LIN_GLU>(a, 1, (hipStream_t)stream);
  } else {
    fstu_set_error("fstu_glu_decode: unknown dtype %d", dtype);
    return FSTU_EDTYPE;
  }
  FSTU_CHECK_LAUNCH("fstu_glu_decode");
  return FSTU_OK;
}

extern "C" int fstu_linear_decode_splitk(const void* x, int ldx, const void* W, float* partial, int rows, int N, int K,
                                         int ksplit, int dtype, void* stream) {
  int rc = check_common("fstu_linear_decode_splitk", x, W, partial, ldx, rows, N, K);
  if (rc) return rc;
  FSTU_REQUIRE(ksplit >= 1 && ksplit <= 1024 && ksplit <= K, FSTU_EARG, "fstu_linear_decode_splitk: ksplit=%d", ksplit);
  LinArgs a{x, ldx, W, nullptr, partial, N, rows, N, K, K, nullptr, 1.0f};
  if (dtype == FSTU_BF16) {
    if (mfma_ok(x, ldx, W, nullptr, K, ksplit)) launch_mfma<LIN_PARTIAL>(a, ksplit, (hipStream_t)stream);
    else launch_valu<bf16_t, LIN_PARTIAL>(a, ksplit, (hipStream_t)stream);
  } else if (dtype == FSTU_F32) {
    launch_valu<float, LIN_PARTIAL>(a, ksplit, (hipStream_t)stream);
  } else {
    fstu_set_error("fstu_linear_decode_splitk: unknown dtype %d", dtype);
    return FSTU_EDTYPE;
  }
  FSTU_CHECK_LAUNCH("fstu_linear_decode_splitk");
  return FSTU_OK;
}

// ---------------------------------------------------------------- head with fused greedy pick
__global__ void __launch_bounds__(1024)
argmax_finish_kernel(unsigned long long* best, int64_t* tok_out, int64_t stride, int rows, int* dyn, int advance) {
  // one workgroup, one wave per row: maximum over the 64 slots, which are cleared for the next call; with
  // `advance` the position/step counters are bumped once every row has used them
  const int b = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = dyn ? dyn[0] : 0;
  __syncthreads();
  if (threadIdx.x == 0 && dyn && advance) { dyn[0] = pos + 1; dyn[1] += 1; }
  if (b >= rows) return;
  unsigned long long k = best[(size_t)b * 64 + lane];
  best[(size_t)b * 64 + lane] = 0ull;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    unsigned long long t = __shfl_xor(k, o, FSTU_WAVE);
    k = t > k ? t : k;
  }
  if (lane == 0) tok_out[(size_t)b * stride + pos] = (int64_t)(0xffffffffu - (unsigned)(k & 0xffffffffull));
}

int fstu_argmax_finish_launch(void* best_ws, int64_t* tok_out, int64_t tok_stride, int rows, int* dyn, int advance, void* stream) {
  hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(rows * 64), 0, (hipStream_t)stream, (unsigned long long*)best_ws,
                     tok_out, tok_stride, rows, dyn, advance);
  FSTU_CHECK_LAUNCH("argmax_finish");
  return FSTU_OK;
}

extern "C" int fstu_head_argmax(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                                float temperature, void* best_ws, int64_t* tok_out, int64_t tok_stride, int dtype,
                                void* stream) {
  return fstu_head_argmax_dyn(x, ldx, W, logits, ldy, rows, N, K, temperature, best_ws, tok_out, tok_stride, nullptr, 0,
                              dtype, stream);
}

// true when fstu_head_argmax takes the path that leaves packed maxima in the workspace (and so can defer their reduction)
bool fstu_head_argmax_fused_pick(const void* x, int ldx, const void* W, int K, int dtype) {
  return dtype == FSTU_BF16 && mfma_ok(x, ldx, W, nullptr, K, 1);
}

int fstu_head_argmax_dyn(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                         float temperature, void* best_ws, int64_t* tok_out, int64_t tok_stride, int* dyn, int advance,
                         int dtype, void* stream) {
  int rc = check_common("fstu_head_argmax", x, W, logits, ldx, rows, N, K);
  if (rc) return rc;
  FSTU_REQUIRE(best_ws && tok_out, FSTU_ENULL, "fstu_head_argmax: null workspace or output");
  FSTU_REQUIRE(ldy >= N && tok_stride >= 1 && temperature > 0.f, FSTU_EARG, "fstu_head_argmax: bad ldy / stride / temperature");
  FSTU_REQUIRE(fstu_aligned(best_ws, 8), FSTU_EALIGN, "fstu_head_argmax: workspace must be 8-byte aligned");
  if (dtype == FSTU_BF16 && mfma_ok(x, ldx, W, nullptr, K, 1)) {
    LinArgs a{x, ldx, W, nullptr, logits, ldy, rows, N, K, K, (unsigned long long*)best_ws, temperature};
    launch_mfma<LIN_ARGMAX>(a, 1, (hipStream_t)stream);
    // advance < 0: the caller's next launch reduces the maxima itself (fstu_finish_embed_rmsnorm)
    if (advance >= 0)
      hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(rows * 64), 0, (hipStream_t)stream, (unsigned long long*)best_ws,
                         tok_out, tok_stride, rows, dyn, advance);
    FSTU_CHECK_LAUNCH("fstu_head_argmax");
    return FSTU_OK;
  }
  rc = fstu_linear_decode(x, ldx, W, logits, ldy, rows, N, K, dtype, stream);
  if (rc) return rc;
  FSTU_REQUIRE(ldy == N, FSTU_ESHAPE, "fstu_head_argmax: this dtype/shape needs dense logits (ldy == N)");
  rc = fstu_sample_dyn(logits, tok_out, tok_stride, rows, N, temperature, 0, 0.f, 0, 0, 0, 0, dyn, dtype, stream);
  if (rc == 0 && dyn && advance) rc = fstu_advance_dyn(dyn, stream);
  return rc;
}

extern "C" int fstu_head_maxima(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                                float temperature, void* best_ws, int dtype, void* stream) {
  int rc = check_common("fstu_head_maxima", x, W, logits, ldx, rows, N, K);
  if (rc) return rc;
  FSTU_REQUIRE(best_ws, FSTU_ENULL, "fstu_head_maxima: null workspace");
  FSTU_REQUIRE(ldy >= N && temperature > 0.f, FSTU_EARG, "fstu_head_maxima: bad ldy / temperature");
  FSTU_REQUIRE(fstu_aligned(best_ws, 8), FSTU_EALIGN, "fstu_head_maxima: workspace must be 8-byte aligned");
  FSTU_REQUIRE(fstu_head_argmax_fused_pick(x, ldx, W, K, dtype), FSTU_ESHAPE,
               "fstu_head_maxima: needs bf16, K %% 256 == 0 and 16-byte aligned rows");
  LinArgs a{x, ldx, W, nullptr, logits, ldy, rows, N, K, K, (unsigned long long*)best_ws, temperature};
  launch_mfma<LIN_ARGMAX>(a, 1, (hipStream_t)stream);
  FSTU_CHECK_LAUNCH("fstu_head_maxima");
  return FSTU_OK;
}

// ---------------------------------------------------------------- head + greedy pick without any allocation
// The packed per-row maxima of the head kernel live in a file-scope device array instead of a caller workspace, for
// callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid hipMalloc).  Every GPU
// holds its own copy of the array at its own address; the host only ever uses the address hipGetSymbolAddress returns
// for the current device, never the array's name.
#define FSTU_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned long long scratch[FSTU_MAX_DECODE_ROWS * 64];   // 8 KiB per GPU
static unsigned long long* g_scratch_ptr[FSTU_STATIC_MAX_DEVICES];   // per device, filled on first use
static std::mutex g_scratch_mu;

__global__ void __launch_bounds__(1024) fill_zero_u64_kernel(unsigned long long* p, int n) {
  const int i = blockIdx.x * 1024 + threadIdx.x;
  if (i < n) p[i] = 0ull;
}

static int static_scratch(unsigned long long** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { fstu_set_error("fstu_head_argmax_static: hipGetDevice: %s", hipGetErrorString(e)); return (int)e; }
  FSTU_REQUIRE(dev >= 0 && dev < FSTU_STATIC_MAX_DEVICES, FSTU_EARG, "fstu_head_argmax_static: device index %d outside 0..%d", dev,
               FSTU_STATIC_MAX_DEVICES - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fstu_set_error("fstu_head_argmax_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return e != hipSuccess ? (int)e : FSTU_EARG;
    }
    g_scratch_ptr[dev] = (unsigned long long*)p;
  }
  *out = g_scratch_ptr[dev];
  return FSTU_OK;
}

extern "C" int fstu_head_argmax_static(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                                       float temperature, int64_t* tok_out, int64_t tok_stride, int dtype, void* stream) {
  FSTU_REQUIRE(rows >= 1 && rows <= FSTU_MAX_DECODE_ROWS, FSTU_ESHAPE,
               "fstu_head_argmax_static: rows=%d beyond the static scratch (%d rows x 64 slots)", rows, FSTU_MAX_DECODE_ROWS);
  unsigned long long* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc) return rc;
  // the array keeps whatever the last call on this GPU left (an interrupted call may have left maxima behind)
  hipLaunchKernelGGL(fill_zero_u64_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ws, FSTU_MAX_DECODE_ROWS * 64);
  FSTU_CHECK_LAUNCH("fstu_head_argmax_static");
  return fstu_head_argmax_dyn(x, ldx, W, logits, ldy, rows, N, K, temperature, ws, tok_out, tok_stride, nullptr, 0, dtype,
                              stream);
}
