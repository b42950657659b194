// Spectral convolution of the STU prefill as the reference computes it (rfft -> product -> irfft,
// flash_stu/utils/stu_utils.py:195-246), as in-LDS complex FFTs on gfx950.
//
// One workgroup transforms `cols` whole columns (one (batch, channel) signal each) that live in LDS from the
// first load to the last store: forward decimation-in-frequency passes (natural order in, digit-reversed order
// out), a pointwise product with a filter spectrum stored in that same digit-reversed order, and the mirrored
// decimation-in-time passes back to natural order.  No bit-reversal pass is ever needed.  A pass is a radix-16
// (first pass: 2, 4, 8 or 16) butterfly held in registers, so a length-4096 transform touches LDS three times.
//
// Both sign branches come out of ONE inverse transform: with F the filter's spectrum, the minus branch
// conv(x, (-1)^s f) has spectrum F[k + n/2], so the product X * (F[k] + i F[k + n/2]) inverts to
// plus + i*minus (both real).  k + n/2 sits at digit-reversed position p ^ 8 because the last pass has radix 16.
#include "fstu_common.h"

namespace {

typedef float2 cpx;

__device__ __forceinline__ cpx cadd(cpx a, cpx b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ cpx csub(cpx a, cpx b) { return make_float2(a.x - b.x, a.y - b.y); }
__device__ __forceinline__ cpx cmul(cpx a, cpx b) {
  return make_float2(fmaf(a.x, b.x, -a.y * b.y), fmaf(a.x, b.y, a.y * b.x));
}
// a * conj(b)
__device__ __forceinline__ cpx cmulc(cpx a, cpx b) {
  return make_float2(fmaf(a.x, b.x, a.y * b.y), fmaf(a.y, b.x, -a.x * b.y));
}
__device__ __forceinline__ cpx cconj(cpx a) { return make_float2(a.x, -a.y); }

// LDS index of element i of a column: one pad slot every 16 elements keeps the stride-16 accesses of the
// last pass (and every other power-of-two stride) off a single bank.
__device__ __forceinline__ int phys(int i) { return i + (i >> 4); }

// z * exp(-2 pi i k / 16), k = 0..7, k known at compile time after unrolling
__device__ __forceinline__ cpx mul_root16(cpx z, int k) {
  const float s = 0.70710678118654752f, c1 = 0.92387953251128674f, s1 = 0.38268343236508977f;
  switch (k) {
    case 0: return z;
    case 1: return make_float2(fmaf(c1, z.x, s1 * z.y), fmaf(c1, z.y, -s1 * z.x));
    case 2: return make_float2((z.x + z.y) * s, (z.y - z.x) * s);
    case 3: return make_float2(fmaf(s1, z.x, c1 * z.y), fmaf(s1, z.y, -c1 * z.x));
    case 4: return make_float2(z.y, -z.x);
    case 5: return make_float2(fmaf(-s1, z.x, c1 * z.y), fmaf(-s1, z.y, -c1 * z.x));
    case 6: return make_float2((z.y - z.x) * s, -(z.x + z.y) * s);
    default: return make_float2(fmaf(-c1, z.x, s1 * z.y), fmaf(-c1, z.y, -s1 * z.x));
  }
}

template <int R> __device__ __forceinline__ constexpr int brev(int k) {
  int r = 0;
  for (int b = 1; b < R; b <<= 1) {
    r = (r << 1) | (k & 1);
    k >>= 1;
  }
  return r;
}

// In-register DFT of R points (R = 2, 4, 8, 16): input v[m] in natural order, output k left in v[brev(k)].
template <int R> __device__ __forceinline__ void dft_inreg(cpx (&v)[R]) {
#pragma unroll
  for (int h = R / 2; h >= 1; h >>= 1) {
#pragma unroll
    for (int b0 = 0; b0 < R; b0 += 2 * h) {
#pragma unroll
      for (int j = 0; j < h; ++j) {
        cpx a = v[b0 + j], b = v[b0 + j + h];
        v[b0 + j] = cadd(a, b);
        v[b0 + j + h] = mul_root16(csub(a, b), j * (8 / h));
      }
    }
  }
}

// a * exp(-2 pi i k / 16) for a real a (the values mul_root16 gives for z = (a, 0))
__device__ __forceinline__ cpx mul_root16_real(float a, int k) {
  const float s = 0.70710678118654752f, c1 = 0.92387953251128674f, s1 = 0.38268343236508977f;
  switch (k) {
    case 0: return make_float2(a, 0.f);
    case 1: return make_float2(c1 * a, -s1 * a);
    case 2: return make_float2(a * s, -a * s);
    case 3: return make_float2(s1 * a, -c1 * a);
    case 4: return make_float2(0.f, -a);
    case 5: return make_float2(-s1 * a, -c1 * a);
    case 6: return make_float2(-a * s, -a * s);
    default: return make_float2(-c1 * a, -s1 * a);
  }
}

// The R-point DFT of a real input whose upper half is zero (a zero-padded signal in the first pass of its transform):
// the first stage adds and subtracts nothing, v[j + R/2] = x[j] W_R^j, and the other stages run as always.
// in: x[0 .. R/2) ; out: as dft_inreg.
template <int R> __device__ __forceinline__ void dft_inreg_real_half(const float (&x)[R / 2], cpx (&v)[R]) {
#pragma unroll
  for (int j = 0; j < R / 2; ++j) {
    v[j] = make_float2(x[j], 0.f);
    v[j + R / 2] = mul_root16_real(x[j], j * (16 / R));
  }
#pragma unroll
  for (int h = R / 4; h >= 1; h >>= 1) {
#pragma unroll
    for (int b0 = 0; b0 < R; b0 += 2 * h) {
#pragma unroll
      for (int j = 0; j < h; ++j) {
        cpx a = v[b0 + j], b = v[b0 + j + h];
        v[b0 + j] = cadd(a, b);
        v[b0 + j + h] = mul_root16(csub(a, b), j * (8 / h));
      }
    }
  }
}

// powers 1..R-1 of w = tw[r*ts] : the binary powers come from the table, the rest are products of two of them
template <int R> __device__ __forceinline__ void twiddle_powers(cpx (&pw)[R], const cpx* __restrict__ tw, int e) {
  pw[0] = make_float2(1.f, 0.f);
  pw[1] = tw[e];
  if (R >= 4) {
    pw[2] = tw[2 * e];
    pw[3] = cmul(pw[1], pw[2]);
  }
  if (R >= 8) {
    pw[4] = tw[4 * e];
    pw[5] = cmul(pw[4], pw[1]);
    pw[6] = cmul(pw[4], pw[2]);
    pw[7] = cmul(pw[4], pw[3]);
  }
  if (R >= 16) {
    pw[8] = tw[8 * e];
#pragma unroll
    for (int k = 1; k < 8; ++k) pw[8 + k] = cmul(pw[8], pw[k]);
  }
}

template <int R> __host__ __device__ constexpr int lg_radix() { return R == 16 ? 4 : R == 8 ? 3 : R == 4 ? 2 : 1; }

// One radix-R butterfly of a pass over blocks of Nb = R*q elements (q = 1 << LQ).  Forward: decimation in
// frequency, y[k] = w^(r k) * sum_m x[m] W_R^(m k) written where x was read.  Inverse: the exact mirror.
// The transform length and the stride are compile-time constants: the R points of a butterfly sit a fixed distance
// apart in the padded column (q + q/16 slots; q = 1 only occurs with R = 16 on blocks that start at a multiple of
// 16), so their addresses are one base and immediate offsets.
// HALF 1 (forward, first pass of a transform): the inputs are real and the upper half of the column is zero (a signal
// of at most n/2 samples): only the lower half's real parts are read.  HALF 2 (inverse, last pass): only the lower
// half of the column is wanted afterwards, the other outputs are neither stored nor (their last stage) computed.
template <int R, bool INV, int LQ, int LOGN, int HALF = 0>
__device__ __forceinline__ void butterfly(cpx* __restrict__ col, const cpx* __restrict__ tw, int u) {
  static_assert(HALF == 0 || (HALF == 1 && !INV) || (HALF == 2 && INV), "half-column passes: forward first, inverse last");
  static_assert(HALF == 0 || LQ + lg_radix<R>() == LOGN, "half-column passes span the whole column");
  constexpr int LR = lg_radix<R>();
  constexpr int q = 1 << LQ;
  constexpr int TS = 1 << (LOGN - LQ - LR);   // table stride: w_Nb = tw[TS]
  constexpr int ST = (LQ >= 4) ? (q + (q >> 4)) : 1;
  static_assert(LQ == 0 || LQ >= 4, "strides between 2 and 8 would cross a pad slot");
  const int r = u & (q - 1);
  const int base = ((u >> LQ) << (LQ + LR)) + r;
  cpx* __restrict__ p = col + phys(base);
  cpx v[R], pw[R];
  constexpr bool twid = LQ > 0;
  if (twid) twiddle_powers<R>(pw, tw, r * TS);
  if (!INV) {
    if constexpr (HALF == 1) {
      float xr[R / 2];
#pragma unroll
      for (int m = 0; m < R / 2; ++m) xr[m] = p[m * ST].x;
      dft_inreg_real_half<R>(xr, v);
    } else {
#pragma unroll
      for (int m = 0; m < R; ++m) v[m] = p[m * ST];
      dft_inreg<R>(v);
    }
#pragma unroll
    for (int k = 0; k < R; ++k) {
      cpx o = v[brev<R>(k)];
      if (twid && k > 0) o = cmul(o, pw[k]);
      p[k * ST] = o;
    }
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k) {
      cpx o = p[k * ST];
      if (twid && k > 0) o = cmulc(o, pw[k]);
      v[k] = cconj(o);
    }
    dft_inreg<R>(v);
#pragma unroll
    for (int m = 0; m < (HALF == 2 ? R / 2 : R); ++m) p[m * ST] = cconj(v[brev<R>(m)]);
  }
}

template <int LOGN> __host__ __device__ constexpr int col_stride() { return (1 << LOGN) + (1 << (LOGN - 4)); }

template <int R, bool INV, int LQ, int LOGN, int NT, int HALF = 0>
__device__ __forceinline__ void run_pass(cpx* lds, const cpx* __restrict__ tw, int cols) {
  constexpr int LPER = LOGN - lg_radix<R>();   // log2 of butterflies per column
  const int total = cols << LPER;
  for (int w = threadIdx.x; w < total; w += NT)
    butterfly<R, INV, LQ, LOGN, HALF>(lds + (size_t)(w >> LPER) * col_stride<LOGN>(), tw, w & ((1 << LPER) - 1));
  __syncthreads();
}

// LOGN = 4*a + rem: the first forward pass has radix 2^rem (if rem > 0), every other pass radix 16.  The last forward
// pass and the first inverse pass work on the same 16 neighbours of a column (stride 1): callers that multiply by a
// spectrum in between skip both here and do the three steps in registers (fft_middle).
// HALF_COL: the columns hold real signals of at most n/2 samples (forward: the pass that spans the whole column reads
// only those; inverse: only the lower half of the result is produced).
// NO_R2 (lengths with a radix-2 pass): the caller performs that pass itself while it writes the column (forward) or
// collects the results (inverse).
template <int LOGN, int NT, bool SKIP_LAST, bool HALF_COL = false, bool NO_R2 = false>
__device__ __forceinline__ void fft_forward(cpx* lds, const cpx* __restrict__ tw, int cols) {
  constexpr int REM = LOGN & 3, TOP = LOGN - REM;
  constexpr int H = HALF_COL ? 1 : 0;
  constexpr int H16A = (REM == 0 && TOP == 12) ? H : 0, H16B = (REM == 0 && TOP == 8) ? H : 0;
  if constexpr (REM == 1 && !NO_R2) run_pass<2, false, LOGN - 1, LOGN, NT, H>(lds, tw, cols);
  if constexpr (REM == 2) run_pass<4, false, LOGN - 2, LOGN, NT, H>(lds, tw, cols);
  if constexpr (REM == 3) run_pass<8, false, LOGN - 3, LOGN, NT, H>(lds, tw, cols);
  if constexpr (TOP >= 12) run_pass<16, false, 8, LOGN, NT, H16A>(lds, tw, cols);
  if constexpr (TOP >= 8) run_pass<16, false, 4, LOGN, NT, H16B>(lds, tw, cols);
  if constexpr (!SKIP_LAST) run_pass<16, false, 0, LOGN, NT>(lds, tw, cols);
}

template <int LOGN, int NT, bool SKIP_FIRST, bool HALF_COL = false, bool NO_R2 = false>
__device__ __forceinline__ void fft_inverse(cpx* lds, const cpx* __restrict__ tw, int cols) {
  constexpr int REM = LOGN & 3, TOP = LOGN - REM;
  constexpr int H = HALF_COL ? 2 : 0;
  constexpr int H16A = (REM == 0 && TOP == 12) ? H : 0, H16B = (REM == 0 && TOP == 8) ? H : 0;
  if constexpr (!SKIP_FIRST) run_pass<16, true, 0, LOGN, NT>(lds, tw, cols);
  if constexpr (TOP >= 8) run_pass<16, true, 4, LOGN, NT, H16B>(lds, tw, cols);
  if constexpr (TOP >= 12) run_pass<16, true, 8, LOGN, NT, H16A>(lds, tw, cols);
  if constexpr (REM == 1 && !NO_R2) run_pass<2, true, LOGN - 1, LOGN, NT, H>(lds, tw, cols);
  if constexpr (REM == 2) run_pass<4, true, LOGN - 2, LOGN, NT, H>(lds, tw, cols);
  if constexpr (REM == 3) run_pass<8, true, LOGN - 3, LOGN, NT, H>(lds, tw, cols);
}

// 16 spectrum values of 16 neighbouring positions (128 contiguous bytes)
__device__ __forceinline__ void load_spec16(const cpx* __restrict__ sp, cpx (&s)[16]) {
#pragma unroll
  for (int k = 0; k < 16; k += 2) {
    const float4 t = *(const float4*)(sp + k);
    s[k] = make_float2(t.x, t.y);
    s[k + 1] = make_float2(t.z, t.w);
  }
}

// forward stride-1 butterfly of 16 neighbours, left in registers in position order (x[k] belongs to position base + k)
__device__ __forceinline__ void forward16(const cpx* __restrict__ p, cpx (&x)[16]) {
  cpx v[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) v[m] = p[m];
  dft_inreg<16>(v);
#pragma unroll
  for (int k = 0; k < 16; ++k) x[k] = v[brev<16>(k)];
}

// x[k] * s[k] through the inverse stride-1 butterfly, written to the 16 neighbours
__device__ __forceinline__ void product_inverse16(cpx* __restrict__ p, const cpx (&x)[16], const cpx (&s)[16]) {
  cpx v[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) v[k] = cconj(cmul(x[k], s[k]));
  dft_inreg<16>(v);
#pragma unroll
  for (int m = 0; m < 16; ++m) p[m] = cconj(v[brev<16>(m)]);
}

// last forward pass, product with the per-column spectra spec[(c0 + col) * n + position], first inverse pass
template <int LOGN, int NT>
__device__ __forceinline__ void fft_middle(cpx* lds, const cpx* __restrict__ spec, int c0, int ncol) {
  constexpr int LPER = LOGN - 4;
  const int total = ncol << LPER;
  for (int w = threadIdx.x; w < total; w += NT) {
    const int colid = w >> LPER, u = w & ((1 << LPER) - 1);
    cpx* p = lds + (size_t)colid * col_stride<LOGN>() + 17 * u;   // phys(16 u)
    cpx s[16], x[16];
    load_spec16(spec + ((size_t)(c0 + colid) << LOGN) + 16 * u, s);
    forward16(p, x);
    product_inverse16(p, x, s);
  }
  __syncthreads();
}

// ---------------------------------------------------------------- twiddle table
__global__ void fft_twiddle_kernel(cpx* __restrict__ tw, int n) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= n) return;
  double s, c;
  sincospi(-2.0 * (double)j / (double)n, &s, &c);
  tw[j] = make_float2((float)c, (float)s);
}

// ---------------------------------------------------------------- filter spectra
// Column j of the filter matrix (element (s, j) at filt[s*f_ls + j*f_cs], taps s < taps) -> spec[j*n + p] =
// (F[p] + i F[p^8]) / n (both branches) or F[p] / n, p running over the digit-reversed positions.
template <typename T, int LOGN, int NT>
__global__ void __launch_bounds__(NT)
fft_filter_kernel(const T* __restrict__ filt, size_t f_ls, size_t f_cs, cpx* __restrict__ spec,
                  const cpx* __restrict__ tw, int taps, int ncol_total, int lcols, int both) {
  extern __shared__ cpx fft_lds[];
  constexpr int n = 1 << LOGN, colstride = col_stride<LOGN>();
  const int cols = 1 << lcols;
  const int c0 = blockIdx.x * cols;
  for (int idx = threadIdx.x; idx < (cols << LOGN); idx += NT) {
    const int colid = idx & (cols - 1), s = idx >> lcols;
    float v = 0.f;
    if (s < taps && c0 + colid < ncol_total) v = DT<T>::ld(filt + (size_t)s * f_ls + (size_t)(c0 + colid) * f_cs);
    fft_lds[(size_t)colid * colstride + phys(s)] = make_float2(v, 0.f);
  }
  __syncthreads();
  fft_forward<LOGN, NT, false>(fft_lds, tw, cols);
  const float inv_n = 1.0f / (float)n;
  for (int idx = threadIdx.x; idx < (cols << LOGN); idx += NT) {
    const int colid = idx >> LOGN, p = idx & (n - 1);
    if (c0 + colid >= ncol_total) continue;
    const cpx* col = fft_lds + (size_t)colid * colstride;
    cpx f = col[phys(p)];
    if (both) {
      const cpx g = col[phys(p ^ 8)];
      f = make_float2(f.x - g.y, f.y + g.x);
    }
    spec[(size_t)(c0 + colid) * n + p] = make_float2(f.x * inv_n, f.y * inv_n);
  }
}

// ---------------------------------------------------------------- convolution
// x element (b, t, c) at x[b*x_sb + t*x_st + c*x_sc]; the K outputs of channel c (K = 1: per-channel spectra
// spec[c]; K > 1: a shared bank spec[k]) go to y[b*y_sb + t*y_st + k*y_sk + c*y_sc] (and y2 likewise).
// mode 0: y = T(T(re) + T(im));  mode 1: y = T(re);  mode 2: y = T(re), y2 = T(im).
template <typename T, int LOGN, int NT>
__global__ void __launch_bounds__(NT)
fft_conv_kernel(const T* __restrict__ x, size_t x_sb, size_t x_st, size_t x_sc, const cpx* __restrict__ spec,
                T* __restrict__ y, T* __restrict__ y2, size_t y_sb, size_t y_st, size_t y_sk, size_t y_sc,
                const cpx* __restrict__ tw, int Tn, int d, int K, int lcols, int mode, int xcd_remap) {
  extern __shared__ cpx fft_lds[];
  constexpr int n = 1 << LOGN, colstride = col_stride<LOGN>();
  const int cols = 1 << lcols;
  int bx = blockIdx.x;
  if (xcd_remap) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);   // consecutive channel groups share an XCD
  const int c0 = bx * cols;
  const int b = blockIdx.y;
  const int ncol = min(cols, d - c0);
  const T* xb = x + (size_t)b * x_sb + (size_t)c0 * x_sc;
  const bool t_fast = x_st == 1;   // time-major input: walk t with the lanes

  for (int idx = threadIdx.x; idx < (cols << LOGN); idx += NT) {
    int colid, t;
    if (t_fast) { colid = idx >> LOGN; t = idx & (n - 1); } else { colid = idx & (cols - 1); t = idx >> lcols; }
    float v = 0.f;
    if (t < Tn && colid < ncol) v = DT<T>::ld(xb + (size_t)t * x_st + (size_t)colid * x_sc);
    fft_lds[(size_t)colid * colstride + phys(t)] = make_float2(v, 0.f);
  }
  __syncthreads();
  fft_forward<LOGN, NT, true>(fft_lds, tw, cols);

  const bool yt_fast = y_st == 1;
  if (K == 1) {
    fft_middle<LOGN, NT>(fft_lds, spec, c0, ncol);
    fft_inverse<LOGN, NT, true, true>(fft_lds, tw, cols);   // outputs t < Tn <= n/2 only
    T* yb = y + (size_t)b * y_sb + (size_t)c0 * y_sc;
    T* yb2 = (mode == 2) ? y2 + (size_t)b * y_sb + (size_t)c0 * y_sc : nullptr;
    for (int idx = threadIdx.x; idx < cols * Tn; idx += NT) {
      int colid, t;
      if (yt_fast) { colid = idx / Tn; t = idx - colid * Tn; } else { colid = idx & (cols - 1); t = idx >> lcols; }
      if (colid >= ncol) continue;
      const cpx z = fft_lds[(size_t)colid * colstride + phys(t)];
      const size_t o = (size_t)t * y_st + (size_t)colid * y_sc;
      if (mode == 0) DT<T>::st(yb + o, DT<T>::rnd(z.x) + DT<T>::rnd(z.y));
      else {
        DT<T>::st(yb + o, z.x);
        if (mode == 2) DT<T>::st(yb2 + o, z.y);
      }
    }
    return;
  }

  // filter bank (one column per workgroup): the thread keeps the spectrum of its groups of 16 neighbouring positions
  // in registers and runs, per filter, the product and the first inverse pass from them
  constexpr int NB = ((n >> 4) + NT - 1) / NT;     // groups of 16 per thread
  cpx xs[NB][16];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int u = threadIdx.x + i * NT;
    if (u < (n >> 4)) forward16(fft_lds + 17 * u, xs[i]);
  }
  __syncthreads();
  for (int k = 0; k < K; ++k) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int u = threadIdx.x + i * NT;
      if (u < (n >> 4)) {
        cpx s[16];
        load_spec16(spec + ((size_t)k << LOGN) + 16 * u, s);
        product_inverse16(fft_lds + 17 * u, xs[i], s);
      }
    }
    __syncthreads();
    fft_inverse<LOGN, NT, true, true>(fft_lds, tw, 1);      // outputs t < Tn <= n/2 only
    T* yb = y + (size_t)b * y_sb + (size_t)c0 * y_sc + (size_t)k * y_sk;
    T* yb2 = (mode == 2) ? y2 + (size_t)b * y_sb + (size_t)c0 * y_sc + (size_t)k * y_sk : nullptr;
    for (int t = threadIdx.x; t < Tn; t += NT) {
      const cpx z = fft_lds[phys(t)];
      const size_t o = (size_t)t * y_st;
      if (mode == 0) DT<T>::st(yb + o, DT<T>::rnd(z.x) + DT<T>::rnd(z.y));
      else {
        DT<T>::st(yb + o, z.x);
        if (mode == 2) DT<T>::st(yb2 + o, z.y);
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- convolution, whole 16-byte row pieces per lane
// The same computation for channel-contiguous (B, T, d) operands with d a multiple of the workgroup's channel count:
// a workgroup owns CHW = max(COLS, 16 bytes' worth) neighbouring channels, reads them as 16-byte pieces of the rows
// (all loads in flight at once, kept in registers), transforms COLS of them at a time in LDS, collects the results in
// registers and writes 16-byte pieces of the output rows.  Global accesses are 8 (bf16) or 4 (fp32) channels wide
// instead of COLS; for the long transforms (COLS = 1) that is the difference between 2-byte and 16-byte accesses.
template <typename T> struct RowVec;
template <> struct RowVec<bf16_t> {
  static constexpr int CH = 8;
  template <int E> static __device__ __forceinline__ float get(const unsigned (&w)[4]) {
    return __uint_as_float((E & 1) ? (w[E >> 1] & 0xffff0000u) : (w[E >> 1] << 16));
  }
  template <int E> static __device__ __forceinline__ void put(unsigned (&w)[4], float v) {
    const unsigned h = f32_to_bf16(v);
    w[E >> 1] = (E & 1) ? ((w[E >> 1] & 0x0000ffffu) | (h << 16)) : ((w[E >> 1] & 0xffff0000u) | h);
  }
};
template <> struct RowVec<float> {
  static constexpr int CH = 4;
  template <int E> static __device__ __forceinline__ float get(const unsigned (&w)[4]) { return __uint_as_float(w[E]); }
  template <int E> static __device__ __forceinline__ void put(unsigned (&w)[4], float v) { w[E] = __float_as_uint(v); }
};

// columns in LDS at a time: as many as 34 KB hold (at most 16); n = 4096 takes two with twice the threads (measured
// 14 % faster than one), n = 8192 one (two with 1024 threads spill registers and were 12 % slower)
template <int LOGN> __host__ __device__ constexpr int fft_lcols() { return LOGN >= 13 ? 0 : LOGN == 12 ? 1 : (12 - LOGN > 4 ? 4 : 12 - LOGN); }

// R2: the radix-2 first pass of the forward transform happens here.  Its butterfly pairs sample t with the zero at
// t + n/2, so position t keeps x and position t + n/2 receives x * w^t (wt = tw[t]): the same values the pass would
// leave, without its trip through LDS and its barrier.
template <typename T, int LOGN, int NT, int G, int E, bool R2 = false>
__device__ __forceinline__ void rows_scatter(cpx* lds, const unsigned (&w)[4], int t, int part, cpx wt = make_float2(1.f, 0.f)) {
  constexpr int COLS = 1 << fft_lcols<LOGN>(), CH = RowVec<T>::CH, VR = (COLS > CH ? COLS : CH) / CH;
  constexpr int n = 1 << LOGN;
  if constexpr (E < CH) {
    // VR == 1: the column is known at compile time; VR > 1 (one group): it follows the row piece
    constexpr int col_ct = E - G * COLS;
    if constexpr (VR > 1 || (col_ct >= 0 && col_ct < COLS)) {
      const int col = VR > 1 ? part * CH + E : col_ct;
      const float xv = RowVec<T>::template get<E>(w);
      cpx* c = lds + (size_t)col * col_stride<LOGN>();
      c[phys(t)] = make_float2(xv, 0.f);
      if constexpr (R2) c[phys(t + n / 2)] = make_float2(xv * wt.x, xv * wt.y);
    }
    rows_scatter<T, LOGN, NT, G, E + 1, R2>(lds, w, t, part, wt);
  }
}

// R2: the radix-2 last pass of the inverse transform happens here, for the wanted lower half only:
// y[t] = u[t] + u[t + n/2] * conj(w^t).
template <typename T, int LOGN, int NT, int G, int E, bool R2 = false>
__device__ __forceinline__ void rows_gather(const cpx* lds, unsigned (&w)[4], int t, int part, int mode, cpx wt = make_float2(1.f, 0.f)) {
  constexpr int COLS = 1 << fft_lcols<LOGN>(), CH = RowVec<T>::CH, VR = (COLS > CH ? COLS : CH) / CH;
  constexpr int n = 1 << LOGN;
  if constexpr (E < CH) {
    constexpr int col_ct = E - G * COLS;
    if constexpr (VR > 1 || (col_ct >= 0 && col_ct < COLS)) {
      const int col = VR > 1 ? part * CH + E : col_ct;
      const cpx* c = lds + (size_t)col * col_stride<LOGN>();
      cpx z = c[phys(t)];
      if constexpr (R2) z = cadd(z, cmulc(c[phys(t + n / 2)], wt));
      RowVec<T>::template put<E>(w, mode == 0 ? DT<T>::rnd(z.x) + DT<T>::rnd(z.y) : z.x);
    }
    rows_gather<T, LOGN, NT, G, E + 1, R2>(lds, w, t, part, mode, wt);
  }
}

template <typename T, int LOGN, int NT, int NV, int G>
__device__ __forceinline__ void rows_groups(cpx* lds, const cpx* __restrict__ spec, const cpx* __restrict__ tw,
                                            unsigned (&io)[NV][4], int Tn, int c0, int mode) {
  constexpr int n = 1 << LOGN, COLS = 1 << fft_lcols<LOGN>(), CH = RowVec<T>::CH, CHW = COLS > CH ? COLS : CH;
  constexpr int VR = CHW / CH, NG = CHW / COLS;
  if constexpr (G < NG) {
    if (G > 0) __syncthreads();   // the previous group's results have been collected
    constexpr bool R2 = (LOGN & 3) == 1;   // the radix-2 pass of these lengths rides on the scatter and the gather
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int q = threadIdx.x + r * NT, t = q / VR, part = q % VR;
      if (t < Tn) {
        if constexpr (R2) rows_scatter<T, LOGN, NT, G, 0, true>(lds, io[r], t, part, tw[t]);
        else rows_scatter<T, LOGN, NT, G, 0>(lds, io[r], t, part);
      }
    }
    // zero padding behind the sequence, up to half the column: the first forward pass knows that the upper half of a
    // column is zero and the inputs real and reads neither, the last inverse pass produces the lower half only.
    // (At 512 and 8192 points those passes have radix 2: they are not run at all, the scatter above and the gather
    // below do their work on the way.)
    constexpr bool HF = !R2, HI = !R2;
    constexpr int pad_to = n / 2;
    for (int idx = threadIdx.x; idx < COLS * (pad_to - Tn); idx += NT) {
      const int col = idx / (pad_to - Tn), t = Tn + idx - col * (pad_to - Tn);
      cpx* c = lds + (size_t)col * col_stride<LOGN>();
      c[phys(t)] = make_float2(0.f, 0.f);
      if constexpr (R2) c[phys(t + n / 2)] = make_float2(0.f, 0.f);   // what the radix-2 pass makes of a zero pair
    }
    __syncthreads();
    fft_forward<LOGN, NT, true, HF, R2>(lds, tw, COLS);
    fft_middle<LOGN, NT>(lds, spec, c0 + G * COLS, COLS);
    fft_inverse<LOGN, NT, true, HI, R2>(lds, tw, COLS);
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int q = threadIdx.x + r * NT, t = q / VR, part = q % VR;
      if (t < Tn) {                                   // over the inputs this group consumed
        if constexpr (R2) rows_gather<T, LOGN, NT, G, 0, true>(lds, io[r], t, part, mode, tw[t]);
        else rows_gather<T, LOGN, NT, G, 0>(lds, io[r], t, part, mode);
      }
    }
    rows_groups<T, LOGN, NT, NV, G + 1>(lds, spec, tw, io, Tn, c0, mode);
  }
}

// (8192 points: two workgroups of 512 threads share a compute unit, 70 KB of LDS each, so a thread may hold 128 registers)
template <typename T, int LOGN, int NT>
__global__ void __launch_bounds__(NT, LOGN == 13 ? 4 : 1)
fft_conv_rows_kernel(const T* __restrict__ x, size_t x_sb, size_t x_st, const cpx* __restrict__ spec, T* __restrict__ y,
                     size_t y_sb, size_t y_st, const cpx* __restrict__ tw, int Tn, int mode, int xcd_remap) {
  extern __shared__ cpx fft_lds[];
  constexpr int n = 1 << LOGN, COLS = 1 << fft_lcols<LOGN>(), CH = RowVec<T>::CH, CHW = COLS > CH ? COLS : CH;
  constexpr int VR = CHW / CH, NV = ((n / 2) * VR + NT - 1) / NT;
  int bx = blockIdx.x;
  if (xcd_remap) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);   // consecutive channel groups share an XCD
  const int c0 = bx * CHW, b = blockIdx.y;
  const T* xb = x + (size_t)b * x_sb + c0;
  // the row pieces: inputs at first, each channel's result written over its input once its group is through
  unsigned io[NV][4];
#pragma unroll
  for (int r = 0; r < NV; ++r) {
    const int q = threadIdx.x + r * NT, t = q / VR, part = q % VR;
    // rows behind the sequence re-read its last row (no branch around the load) and are never used
    const uint4 v = *(const uint4*)(xb + (size_t)min(t, Tn - 1) * x_st + part * CH);
    io[r][0] = v.x; io[r][1] = v.y; io[r][2] = v.z; io[r][3] = v.w;
  }
  rows_groups<T, LOGN, NT, NV, 0>(fft_lds, spec, tw, io, Tn, c0, mode);
  T* yb = y + (size_t)b * y_sb + c0;
#pragma unroll
  for (int r = 0; r < NV; ++r) {
    const int q = threadIdx.x + r * NT, t = q / VR, part = q % VR;
    if (t < Tn) *(uint4*)(yb + (size_t)t * y_st + part * CH) = make_uint4(io[r][0], io[r][1], io[r][2], io[r][3]);
  }
}

int ilog2_exact(int n) {
  int l = 0;
  while ((1 << l) < n) ++l;
  return ((1 << l) == n) ? l : -1;
}

// columns per workgroup and threads per workgroup for a transform length
void fft_shape(int logn, int ncol_total, int* lcols, int* nt) {
  int lc = 12 - logn;           // cols * n = 4096 complex elements = 34 KB of LDS
  if (lc < 0) lc = 0;
  if (lc > 4) lc = 4;
  while (lc > 0 && (1 << lc) > ncol_total) --lc;
  *lcols = lc;
  *nt = (logn >= 14) ? 1024 : (logn == 13 ? 512 : 256);
}

size_t fft_lds_bytes(int n, int lcols) { return (size_t)(n + (n >> 4)) * sizeof(cpx) << lcols; }

template <typename K> int allow_lds(K kernel, size_t bytes, const char* name) {
  if (bytes <= 48 * 1024) return 0;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)bytes);
  if (e != hipSuccess) {
    fstu_set_error("%s: %zu bytes of LDS refused: %s", name, bytes, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

}  // namespace

extern "C" int fstu_fft_length(int T_) {
  int n = 64;
  while (n < 2 * T_ && n < (1 << 14)) n <<= 1;
  return (n >= 2 * T_) ? n : 0;
}

extern "C" int fstu_fft_twiddles(float* tw, int n, void* stream) {
  FSTU_REQUIRE(tw, FSTU_ENULL, "fstu_fft_twiddles: null pointer");
  const int logn = ilog2_exact(n);
  FSTU_REQUIRE(logn >= 6 && logn <= 14, FSTU_ESHAPE, "fstu_fft_twiddles: n=%d is not a power of two in 64..16384", n);
  hipLaunchKernelGGL(fft_twiddle_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, (cpx*)tw, n);
  FSTU_CHECK_LAUNCH("fstu_fft_twiddles");
  return FSTU_OK;
}

// threads per workgroup follow the transform length: one radix-16 butterfly per thread and pass for n = 4096 and
// 8192, two at 16384 (1024 threads leave 128 registers each, which the bank form's resident spectrum overflows)
#ifndef FFT_NT14
#define FFT_NT14 512
#endif
#define FFT_LAUNCH_ONE(LOGNV, NTV, KERNEL, GRID, SHM, NAME, ...)                                              \
  do {                                                                                                        \
    int rc__ = allow_lds(KERNEL<T, LOGNV, NTV>, SHM, NAME);                                                   \
    if (rc__) return rc__;                                                                                    \
    hipLaunchKernelGGL((KERNEL<T, LOGNV, NTV>), GRID, dim3(NTV), SHM, (hipStream_t)stream, __VA_ARGS__);      \
  } while (0)

#define FFT_LAUNCH(LOGN, KERNEL, GRID, SHM, NAME, ...)                                  \
  do {                                                                                  \
    switch (LOGN) {                                                                     \
      case 6: FFT_LAUNCH_ONE(6, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 7: FFT_LAUNCH_ONE(7, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 8: FFT_LAUNCH_ONE(8, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 9: FFT_LAUNCH_ONE(9, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 10: FFT_LAUNCH_ONE(10, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 11: FFT_LAUNCH_ONE(11, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 12: FFT_LAUNCH_ONE(12, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 13: FFT_LAUNCH_ONE(13, 512, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      default: FFT_LAUNCH_ONE(14, FFT_NT14, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;   \
    }                                                                                   \
  } while (0)

#define FFT_LAUNCH_ROWS(LOGN, KERNEL, GRID, SHM, NAME, ...)                              \
  do {                                                                                  \
    switch (LOGN) {                                                                     \
      case 6: FFT_LAUNCH_ONE(6, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 7: FFT_LAUNCH_ONE(7, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 8: FFT_LAUNCH_ONE(8, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 9: FFT_LAUNCH_ONE(9, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;      \
      case 10: FFT_LAUNCH_ONE(10, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 11: FFT_LAUNCH_ONE(11, 256, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 12: FFT_LAUNCH_ONE(12, 512, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      case 13: FFT_LAUNCH_ONE(13, 512, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
      default: FFT_LAUNCH_ONE(14, 512, KERNEL, GRID, SHM, NAME, __VA_ARGS__); break;    \
    }                                                                                   \
  } while (0)

extern "C" int fstu_stu_fft_filter(const void* filt, int64_t f_ls, int64_t f_cs, float* spec, const float* tw, int taps,
                                   int ncols, int n, int single_branch, int dtype, void* stream) {
  FSTU_REQUIRE(filt && spec && tw, FSTU_ENULL, "fstu_stu_fft_filter: null pointer");
  const int logn = ilog2_exact(n);
  FSTU_REQUIRE(logn >= 6 && logn <= 14, FSTU_ESHAPE, "fstu_stu_fft_filter: n=%d is not a power of two in 64..16384", n);
  FSTU_REQUIRE(taps >= 1 && 2 * taps <= n && ncols >= 1, FSTU_ESHAPE,
               "fstu_stu_fft_filter: taps=%d must satisfy 1 <= taps <= n/2=%d (ncols=%d)", taps, n / 2, ncols);
  FSTU_REQUIRE(fstu_aligned(spec, 8) && fstu_aligned(tw, 8), FSTU_EALIGN, "fstu_stu_fft_filter: spec/tw must be 8-byte aligned");
  int lcols, nt;
  fft_shape(logn, ncols, &lcols, &nt);
  const size_t shm = fft_lds_bytes(n, lcols);
  dim3 grid((ncols + (1 << lcols) - 1) >> lcols);
  FSTU_DISPATCH_DTYPE(dtype, "fstu_stu_fft_filter",
                      FFT_LAUNCH(logn, fft_filter_kernel, grid, shm, "fstu_stu_fft_filter", (const T*)filt, (size_t)f_ls,
                                 (size_t)f_cs, (cpx*)spec, (const cpx*)tw, taps, ncols, lcols, single_branch ? 0 : 1));
  FSTU_CHECK_LAUNCH("fstu_stu_fft_filter");
  return FSTU_OK;
}

static int conv_fft_launch(const char* name, const void* x, int64_t x_sb, int64_t x_st, int64_t x_sc, const float* spec,
                           void* y, void* y2, int64_t y_sb, int64_t y_st, int64_t y_sk, int64_t y_sc, const float* tw,
                           int B, int T_, int d, int K, int n, int mode, int dtype, void* stream) {
  const int logn = ilog2_exact(n);
  FSTU_REQUIRE(logn >= 6 && logn <= 14, FSTU_ESHAPE, "%s: n=%d is not a power of two in 64..16384", name, n);
  FSTU_REQUIRE(B >= 1 && B <= 65535 && T_ >= 1 && d >= 1 && K >= 1 && 2 * T_ <= n, FSTU_ESHAPE,
               "%s: bad shape B=%d T=%d d=%d K=%d n=%d (n >= 2T required)", name, B, T_, d, K, n);
  FSTU_REQUIRE(fstu_aligned(spec, 8) && fstu_aligned(tw, 8), FSTU_EALIGN, "%s: spec/tw must be 8-byte aligned", name);
  int lcols, nt;
  fft_shape(logn, d, &lcols, &nt);
  if (K > 1) lcols = 0;
  {
    // channel-contiguous operands whose rows split into whole 16-byte pieces per workgroup: the row-piece kernel
    const int rows_lcols = logn >= 13 ? 0 : logn == 12 ? 1 : (12 - logn > 4 ? 4 : 12 - logn);
    const int esz = dtype == FSTU_BF16 ? 2 : 4, ch = 16 / esz, cols_full = 1 << rows_lcols;
    const int chw = cols_full > ch ? cols_full : ch;
    // (the long transforms take a workgroup's channels one after the other: with fewer than two workgroups per compute
    // unit the one-column kernel, eight times the workgroups, is the faster one)
    const bool enough = logn < 13 || (long long)(d / chw) * B >= 512;
    if (K == 1 && mode != 2 && enough && x_sc == 1 && y_sc == 1 && d % chw == 0 && x_st % ch == 0 && y_st % ch == 0 &&
        x_sb % ch == 0 && y_sb % ch == 0 && fstu_aligned(x, 16) && fstu_aligned(y, 16)) {
      const size_t shm = fft_lds_bytes(n, rows_lcols);
      const int gx = d / chw;
      dim3 grid(gx, B);
      const int remap = (gx % 8 == 0) ? 1 : 0;
      FSTU_DISPATCH_DTYPE(dtype, name,
                          FFT_LAUNCH_ROWS(logn, fft_conv_rows_kernel, grid, shm, name, (const T*)x, (size_t)x_sb, (size_t)x_st,
                                          (const cpx*)spec, (T*)y, (size_t)y_sb, (size_t)y_st, (const cpx*)tw, T_, mode, remap));
      FSTU_CHECK_LAUNCH(name);
      return FSTU_OK;
    }
  }
  (void)nt;   // n <= 16 * threads holds for every length: the bank form keeps 16 positions per thread
  const size_t shm = fft_lds_bytes(n, lcols);
  const int gx = (d + (1 << lcols) - 1) >> lcols;
  dim3 grid(gx, B);
  const int remap = (gx % 8 == 0) ? 1 : 0;
  FSTU_DISPATCH_DTYPE(dtype, name,
                      FFT_LAUNCH(logn, fft_conv_kernel, grid, shm, name, (const T*)x, (size_t)x_sb, (size_t)x_st,
                                 (size_t)x_sc, (const cpx*)spec, (T*)y, (T*)y2, (size_t)y_sb, (size_t)y_st, (size_t)y_sk,
                                 (size_t)y_sc, (const cpx*)tw, T_, d, K, lcols, mode, remap));
  FSTU_CHECK_LAUNCH(name);
  return FSTU_OK;
}

extern "C" int fstu_stu_conv_fft(const void* xp, const float* spec, void* y, const float* tw, int B, int T_, int d, int n,
                                 int single_branch, int dtype, void* stream) {
  FSTU_REQUIRE(xp && spec && y && tw, FSTU_ENULL, "fstu_stu_conv_fft: null pointer");
  return conv_fft_launch("fstu_stu_conv_fft", xp, (int64_t)T_ * d, d, 1, spec, y, nullptr, (int64_t)T_ * d, d, 0, 1, tw, B,
                         T_, d, 1, n, single_branch ? 1 : 0, dtype, stream);
}

// The same convolution on strided operands: element (b, t, c) of x at x_strides[0]*b + x_strides[1]*t + x_strides[2]*c
// (elements), y likewise.  Time-major operands (a time stride of 1) make the loads and stores of the one-column
// kernel coalesce, which is what a few long sequences want (few channels x batch rows, transform length 8192 or more).
extern "C" int fstu_stu_conv_fft_strided(const void* xp, const int64_t* x_strides, const float* spec, void* y,
                                         const int64_t* y_strides, const float* tw, int B, int T_, int d, int n,
                                         int single_branch, int dtype, void* stream) {
  FSTU_REQUIRE(xp && x_strides && spec && y && y_strides && tw, FSTU_ENULL, "fstu_stu_conv_fft_strided: null pointer");
  return conv_fft_launch("fstu_stu_conv_fft_strided", xp, x_strides[0], x_strides[1], x_strides[2], spec, y, nullptr, y_strides[0],
                         y_strides[1], 0, y_strides[2], tw, B, T_, d, 1, n, single_branch ? 1 : 0, dtype, stream);
}

extern "C" int fstu_stu_conv_bank_fft(const void* x, const int64_t* x_strides, const float* spec, void* u_plus,
                                      void* u_minus, const int64_t* u_strides, const float* tw, int B, int T_, int d,
                                      int K, int n, int dtype, void* stream) {
  FSTU_REQUIRE(x && x_strides && spec && u_plus && u_strides && tw, FSTU_ENULL, "fstu_stu_conv_bank_fft: null pointer");
  FSTU_REQUIRE(K >= 2, FSTU_ESHAPE, "fstu_stu_conv_bank_fft: K=%d (a bank has at least two filters)", K);
  return conv_fft_launch("fstu_stu_conv_bank_fft", x, x_strides[0], x_strides[1], x_strides[2], spec, u_plus, u_minus,
                         u_strides[0], u_strides[1], u_strides[2], u_strides[3], tw, B, T_, d, K, n, u_minus ? 2 : 1,
                         dtype, stream);
}
