// Prefill sliding-window attention on the matrix cores (bf16), same arithmetic as swa_prefill_kernel:
//   s = softcap*tanh((q.k)*hd^-0.5/softcap) - slope*(p-j) over the keys p-W <= j <= p, softmax in fp32, o = P V
// (flash_stu/modules/attention.py:59-105 with flash-attn's causal window_size=(W,0), alibi_slopes, softcap).
//
// A wave owns 16 consecutive queries of one (batch, head) and walks their keys 32 at a time:
//   S^T (keys x queries) = K Q^T     v_mfma_f32_16x16x32_bf16, K rows straight from the qkv tensor as the A operand;
//                                     the 16 rows of key tile t are the keys 8*(i>>2) + 4*t + (i&3) of the block, so
//                                     that after both tiles lane (g, c) holds the scores of query c against the 8
//                                     CONSECUTIVE keys 8g..8g+7: exactly its B-operand fragment of the second product
//   O^T (dims x queries) = V^T P^T   V^T read from a transposed copy (B,H,hd,Tp) made by swa_vt_kernel, 16 bytes per
//                                     lane; P is split into a bf16 head and a bf16 remainder (two MFMAs), which
//                                     keeps the product at fp32-P accuracy.
// Both products leave query c in lane c of every 16-lane group, so the online-softmax state (max, sum) is per lane
// and rescaling the accumulators needs no cross-lane traffic.
#include "fstu_common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }

// V^T copy: vt[b][h][i][t] = v[b][t][h][i], zero for T <= t < Tp
__global__ void __launch_bounds__(256)
swa_vt_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ vt, int Tn, int Tp, int H, int HD) {
  // a workgroup transposes a 64 (t) x 64 (dims) tile through LDS
  __shared__ bf16_t tile[64][66];
  const int d = H * HD;
  const int t0 = blockIdx.x * 64, i0 = blockIdx.y * 64;   // i over H*HD
  const int b = blockIdx.z;
  for (int e = threadIdx.x; e < 64 * 64; e += 256) {
    const int tt = e >> 6, ii = e & 63;
    bf16_t v = 0;
    if (t0 + tt < Tn && i0 + ii < d) v = qkv[((size_t)b * Tn + t0 + tt) * 3 * d + 2 * d + i0 + ii];
    tile[tt][ii] = v;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 64 * 64; e += 256) {
    const int ii = e >> 6, tt = e & 63;
    if (t0 + tt < Tp && i0 + ii < d) vt[((size_t)b * d + i0 + ii) * Tp + t0 + tt] = tile[tt][ii];
  }
}

template <int HD, int NW>
__global__ void __launch_bounds__(NW * 64)
swa_prefill_mfma_kernel(const bf16_t* __restrict__ qkv, const bf16_t* __restrict__ vt, bf16_t* __restrict__ out,
                        const float* __restrict__ slopes, int Tn, int Tp, int H, int window, float softcap) {
  constexpr int KS = HD / 32;   // k steps of the score product
  constexpr int NT = HD / 16;   // 16-dim tiles of the output
  const int h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int qs = (blockIdx.x * NW + w) * 16;         // first query of this wave
  const bool wave_on = qs < Tn;                      // an idle wave still loads tiles and meets the barriers
  const int d = H * HD;
  const size_t rs = (size_t)3 * d;                   // row stride of qkv
  const bf16_t* base = qkv + (size_t)b * Tn * rs + h * HD;
  const int myq = qs + c;                            // the query whose statistics this lane keeps
  const float scale = rsqrtf((float)HD), slope = slopes[h];
  const float inv_cap2l = softcap > 0.f ? 2.8853900817779268f / softcap : 0.f;   // 2 log2(e) / softcap

  // Q^T fragments (B operand): lane holds Q[query c][dims ks*32 + 8g ..]
  uint4 qf[KS];
  {
    const bf16_t* qr = base + (size_t)min(myq, Tn - 1) * rs + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const uint4*)(qr + ks * 32);
  }
  floatx4_t o[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) o[nt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const int klo = max(0, qs - window);
  const int khi = min(Tn - 1, qs + 15);              // last key any query of the tile may see
  // row i = c of key tile t is key kb + 8*(c>>2) + 4*t + (c&3)
  // The NW waves of a workgroup (16 NW consecutive queries) see nearly the same keys: a block of 32 keys is brought
  // into LDS once for all of them (K rows in the order the MFMA fragments read them, V^T rows; both padded by one
  // 16-byte slot per row so that the 16 rows a quarter wave reads fall on distinct banks), the next block's
  // pieces travel in registers meanwhile.
  constexpr int KCH = HD / 8;                        // 16-byte pieces per key row
  constexpr int NTHR = NW * 64;
  constexpr int KPT = (32 * KCH + NTHR - 1) / NTHR;  // pieces of the K tile per thread
  constexpr int VPT = (HD * 4 + NTHR - 1) / NTHR;    // pieces of the V^T tile per thread
  __shared__ uint4 k_lds[32 * (KCH + 1)];
  __shared__ uint4 v_lds[HD * 5];
  const int qs_wg = blockIdx.x * (NW * 16);
  const int kb_first = (max(0, qs_wg - window) >> 5) << 5;
  const int kb_last = min(Tn - 1, qs_wg + NW * 16 - 1);
  uint4 kreg[KPT], vreg[VPT];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int e = min((int)threadIdx.x + i * NTHR, 32 * KCH - 1), kk = e / KCH, ch = e % KCH;
      kreg[i] = *(const uint4*)(base + (size_t)min(kb + kk, Tn - 1) * rs + d + ch * 8);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = min((int)threadIdx.x + i * NTHR, HD * 4 - 1), dim = e >> 2, ch = e & 3;
      vreg[i] = *(const uint4*)(vt + ((size_t)b * d + h * HD + dim) * Tp + kb + ch * 8);
    }
  };
  fetch(kb_first);
  for (int kb = kb_first; kb <= kb_last; kb += 32) {
    __syncthreads();                                 // the previous block's fragments have been read
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      // (threads beyond the tile's pieces hold a copy of the last piece and store it again: same value, same slot)
      const int e = min((int)threadIdx.x + i * NTHR, 32 * KCH - 1), kk = e / KCH, ch = e % KCH;
      // key kk of the block is row c = 4*(kk>>3) + (kk&3) of key tile t = (kk>>2)&1
      k_lds[(((kk >> 2) & 1) * 16 + 4 * (kk >> 3) + (kk & 3)) * (KCH + 1) + ch] = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = min((int)threadIdx.x + i * NTHR, HD * 4 - 1);
      v_lds[(e >> 2) * 5 + (e & 3)] = vreg[i];
    }
    __syncthreads();
    if (kb + 32 <= kb_last) fetch(kb + 32);
    if (!wave_on || kb > khi || kb + 31 < klo) continue;   // wave-uniform: no key of this block is visible to the wave
    // ---- scores of the block: two key tiles
    floatx4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint4 ka = k_lds[c * (KCH + 1) + ks * 4 + g], kc = k_lds[(16 + c) * (KCH + 1) + ks * 4 + g];
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ka), as_bf16x8(qf[ks]), s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kc), as_bf16x8(qf[ks]), s1, 0, 0, 0);
    }
    uint4 vf[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) vf[nt] = v_lds[(nt * 16 + c) * 5 + g];

    // lane (g, c): D rows 4g+r of tile t are keys kb + 8g + 4t + r, column c is query myq
    float sc[8];
    float bm = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = kb + 8 * g + e;
      float s = (e < 4 ? s0[e] : s1[e - 4]) * scale;
      // soft-cap on the hardware exp2 / reciprocal: tanh(x) = 1 - 2 / (exp(2x) + 1), absolute error about 1e-7 in
      // front of a probability that is rounded to bf16 (the library tanhf costs about 60 instructions per score
      // and was most of this kernel's time)
      if (softcap > 0.f) s = softcap - (2.0f * softcap) * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(s * inv_cap2l) + 1.0f);
      s -= slope * (float)(myq - j);
      const bool valid = j <= myq && j >= myq - window && j < Tn;
      sc[e] = valid ? s : -INFINITY;
      bm = fmaxf(bm, sc[e]);
    }
    bm = fmaxf(bm, fstu_swz16(bm));                       // lane ^ 16
    bm = fmaxf(bm, __shfl_xor(bm, 32, FSTU_WAVE));
    const float mn = fmaxf(m, bm);
    float corr = 1.f;
    unsigned ph[4], pl[4];
    if (mn == -INFINITY) {
#pragma unroll
      for (int e = 0; e < 4; ++e) ph[e] = pl[e] = 0u;
    } else {
      corr = __expf(m - mn);          // m = -inf gives 0
      float p[8];
      float ps = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = __expf(sc[e] - mn);    // masked keys give 0
        ps += p[e];
      }
      l = l * corr + ps;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ph[e] = pack2_bf16(p[2 * e], p[2 * e + 1]);
        pl[e] = pack2_bf16(p[2 * e] - __uint_as_float(ph[e] << 16), p[2 * e + 1] - __uint_as_float(ph[e] & 0xffff0000u));
      }
      m = mn;
    }
    const uint4 pfh = make_uint4(ph[0], ph[1], ph[2], ph[3]), pfl = make_uint4(pl[0], pl[1], pl[2], pl[3]);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) o[nt][r] *= corr;
      o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf[nt]), as_bf16x8(pfh), o[nt], 0, 0, 0);
      o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf[nt]), as_bf16x8(pfl), o[nt], 0, 0, 0);
    }
  }
  // the four lane groups hold disjoint keys: total sum over g
  l += __shfl_xor(l, 16, FSTU_WAVE);
  l += __shfl_xor(l, 32, FSTU_WAVE);
  if (wave_on && myq < Tn) {
    const float inv = 1.0f / l;
    bf16_t* orow = out + ((size_t)b * Tn + myq) * d + h * HD + 4 * g;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      uint2 pk;
      pk.x = pack2_bf16(o[nt][0] * inv, o[nt][1] * inv);
      pk.y = pack2_bf16(o[nt][2] * inv, o[nt][3] * inv);
      *(uint2*)(orow + nt * 16) = pk;
    }
  }
}

}  // namespace

extern "C" int64_t fstu_swa_prefill_ws_elems(int B, int T_, int H, int hd) {
  const int64_t Tp = ((int64_t)T_ + 63) / 64 * 64;
  return (int64_t)B * H * hd * Tp;
}

extern "C" int fstu_swa_prefill_mfma(const void* qkv, void* vt_ws, void* out, const float* slopes, int B, int T_, int H,
                                     int hd, int window, float softcap, void* stream) {
  FSTU_REQUIRE(qkv && vt_ws && out && slopes, FSTU_ENULL, "fstu_swa_prefill_mfma: null pointer");
  FSTU_REQUIRE(B >= 1 && T_ >= 1 && H >= 1 && B <= 65535 && H <= 65535, FSTU_ESHAPE, "fstu_swa_prefill_mfma: bad shape B=%d T=%d H=%d", B, T_, H);
  FSTU_REQUIRE(hd == 64 || hd == 128, FSTU_ESHAPE, "fstu_swa_prefill_mfma: head dim %d not in {64,128}", hd);
  FSTU_REQUIRE(window >= 0, FSTU_EARG, "fstu_swa_prefill_mfma: window<0");
  FSTU_REQUIRE(fstu_aligned(qkv, 16) && fstu_aligned(vt_ws, 16) && fstu_aligned(out, 16), FSTU_EALIGN,
               "fstu_swa_prefill_mfma: pointers must be 16-byte aligned");
  const int Tp = (T_ + 63) / 64 * 64;
  const int d = H * hd;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(swa_vt_kernel, dim3(Tp / 64, (d + 63) / 64, B), dim3(256), 0, s, (const bf16_t*)qkv, (bf16_t*)vt_ws, T_, Tp, H, hd);
  // queries per workgroup (waves sharing one K / V^T tile): 64 at head dim 64, 256 at head dim 128 (measured at
  // 4x1024 tokens, 16 heads of 128, window 1024: 200 us with 4 waves, 130 with 8, 109 with 16; at head dim 64
  // 4 waves were the fastest)
  if (hd == 64) {
    constexpr int NW = 4;
    hipLaunchKernelGGL((swa_prefill_mfma_kernel<64, NW>), dim3((T_ + NW * 16 - 1) / (NW * 16), H, B), dim3(NW * 64), 0, s,
                       (const bf16_t*)qkv, (const bf16_t*)vt_ws, (bf16_t*)out, slopes, T_, Tp, H, window, softcap);
  } else {
    constexpr int NW = 16;
    hipLaunchKernelGGL((swa_prefill_mfma_kernel<128, NW>), dim3((T_ + NW * 16 - 1) / (NW * 16), H, B), dim3(NW * 64), 0, s,
                       (const bf16_t*)qkv, (const bf16_t*)vt_ws, (bf16_t*)out, slopes, T_, Tp, H, window, softcap);
  }
  FSTU_CHECK_LAUNCH("fstu_swa_prefill_mfma");
  return FSTU_OK;
}
