// Prefill GEMMs on the matrix cores (bf16, fp32 accumulation):  C[m, n] = sum_k A[m, k] W[n, k]
// for activations A (M rows, K contiguous) and nn.Linear weights W (N, K) — the dense contractions of the prompt pass
// (c_attn / c_proj flash_stu/modules/attention.py:74,101; gate / up / down flash_stu/modules/swiglu.py:22-29;
// x @ M_inputs flash_stu/modules/stu.py:87), with the element-wise work that follows them as epilogues:
//   mode 0  C = T(acc)
//   mode 1  GLU: C[m, i] = T( T(gelu_tanh(T(acc_gate))) * T(acc_up) ) from two weight matrices (swiglu.py:23-26),
//           so the gate and up activations never travel through HBM
//   mode 2  C = T( R + T(acc) ): the residual add behind c_proj / down_proj (attention_layer.py:57,62, stu_layer.py:96)
//   split-K C = fp32 partial sums per K slice (fstu_add_rmsnorm adds the slices): the down projection of a decode
//           step over 17..32 rows, whose 16 output tiles would leave most of the chip without weights to stream
//
// A workgroup is WFN x WTN waves; a wave owns FI x TJ MFMA tiles of 32 features x 32 rows
// (v_mfma_f32_32x32x16_bf16), the workgroup 32*FI*WFN features x 32*TJ*WTN rows.  K runs in tiles of BK through NS
// LDS stages that are filled straight from global memory (buffer_load_dwordx4 ... lds, no stop in registers) one or more
// tiles ahead of the multiplication.  LDS rows are BK*2 bytes with the 16-byte chunk index XOR-ed with bits of the
// row, so neither the fills nor the fragment reads meet bank conflicts.  The weights are the MFMA A operand and the
// activations the B operand, so a lane ends up with 4 consecutive features of one row: 8-byte stores.  In mode 1 a
// wave's feature tiles are half gate, half up rows of the same features.  Workgroup ids are dealt round-robin to the
// 8 XCDs; each XCD works through its own contiguous share of the tiles in panels of 8 feature tiles, so the workgroups
// resident on an XCD share a few weight and activation tiles in its L2.
#include "fstu_common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

#define GM_PANEL 8     // feature tiles per panel of the tile order
// A workgroup addresses its tile through a buffer descriptor whose base is the tile's first row (64-bit arithmetic) and a
// 32-bit byte offset per lane of at most 256 rows * row stride * 2 bytes: row strides (lda, and K for the weights) stay
// below 2^22 elements so that this offset cannot wrap; what lies beyond a tile's rows is cut off by the descriptor's range
#define GM_MAX_LD (1 << 22)

__device__ __forceinline__ float rnd_bf16(float v) { return bf16_to_f32(f32_to_bf16(v)); }
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  const float e = __builtin_amdgcn_exp2f(2.8853900817779268f * inner);   // exp(2 inner)
  const float th = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
  return 0.5f * x * (1.0f + th);
}

// 16 bytes per lane from global memory into LDS without a stop in registers: the 64 lanes fill 64 consecutive 16-byte
// slots from `l` (wave-uniform) on.  The source is a buffer descriptor (base and range in SGPRs), a 32-bit byte offset
// per lane and a scalar offset for the k tile: rows beyond the range read zeros, so ragged tiles need no clamping
// (measured 2-13 % faster than the same fills through 64-bit per-lane addresses).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (unsigned)bytes, 0x00020000);
}
__device__ __forceinline__ void buf_load16_to_lds(rsrc_t rs, unsigned voff, unsigned soff, void* l) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)l, 16, voff, soff, 0, 0);
}
__device__ __forceinline__ unsigned lds_addr(const void* p) {
  return (unsigned)(size_t)(const __attribute__((address_space(3))) void*)p;
}

// Fragment reads are written as asm: the compiler orders every LDS read it knows of behind all outstanding
// global->LDS loads (s_waitcnt vmcnt(0)), which would serialise the next tile's fetch with this tile's reads.
template <int OFF>
__device__ __forceinline__ u32x4_t lds_read16(unsigned addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int N, int STEP, int I = 0>
__device__ __forceinline__ void lds_read_rows(u32x4_t* f, unsigned addr) {   // N reads, 32 rows (STEP bytes) apart
  if constexpr (I < N) {
    f[I] = lds_read16<I * STEP>(addr);
    lds_read_rows<N, STEP, I + 1>(f, addr);
  }
}
// Waits until at most LEFT of the reads issued so far are outstanding; the fragments pass through the statement so
// that nothing that uses them is placed ahead of the wait.
template <int LEFT, int N>
__device__ __forceinline__ void lds_wait(u32x4_t (&f)[N]) {
  static_assert(N == 3 || N == 4 || N == 6 || N == 8, "fragment group");
  if constexpr (N == 3)
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]) : "n"(LEFT));
  else if constexpr (N == 4)
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]) : "n"(LEFT));
  else if constexpr (N == 6)
    asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]) : "n"(LEFT));
  else
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7])
                 : "n"(LEFT));
}

template <int WFN_, int WTN_, int FI_, int TJ_, int BK_, int NS_>
struct GemmTile {
  static constexpr int WFN = WFN_, WTN = WTN_, FI = FI_, TJ = TJ_, BK = BK_, NS = NS_;
  static constexpr int NW = WFN * WTN, THREADS = 64 * NW;
  static constexpr int BF = 32 * FI * WFN, BT = 32 * TJ * WTN;   // LDS rows of the weight / activation tile
  static constexpr int RB = BK * 2, CPR = RB / 16;               // bytes and 16-byte chunks per LDS row
  static constexpr int KK = BK / 16;                             // MFMA k steps per tile
  static constexpr int WL = BF * CPR / (64 * NW), AL = BT * CPR / (64 * NW);   // fill instructions per wave and tile
  static constexpr unsigned STAGE = (unsigned)(BF + BT) * RB;
  static constexpr unsigned LDS = STAGE * NS;
  static constexpr int NFR = FI + TJ;                            // fragments per k step
  static_assert(BK == 32 || BK == 64, "k tile");
  static_assert((BF * CPR) % (64 * NW) == 0 && (BT * CPR) % (64 * NW) == 0, "fill split");
  // Byte offset of 16-byte chunk c of a row inside a tile.  A 16-byte fragment read is served 16 lanes (16 consecutive
  // rows, one chunk each) at a time and is free of bank conflicts when those 16 pieces fall into 16 different 16-byte
  // slots of a 256-byte window: the row's position inside the window supplies 1 (128-byte rows) or 2 (64-byte rows) of
  // the 4 slot bits, the XOR with the next higher row bits the other 3 or 2.
  __device__ static __forceinline__ unsigned swz(int row, int c) {
    return (unsigned)row * RB + (unsigned)((c ^ (BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3))) << 4);
  }
};

template <class G, int MODE>
__global__ void __launch_bounds__(G::THREADS)
gemm_bf16_kernel(const bf16_t* __restrict__ A, long long lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
                 const bf16_t* __restrict__ R, long long ldr, bf16_t* __restrict__ C, long long ldc, int M, int N, int K,
                 int mt, int nt, int share, int ksplit) {
  constexpr int FI = G::FI, TJ = G::TJ, BF = G::BF, BT = G::BT, WL = G::WL, AL = G::AL, NS = G::NS, KK = G::KK, NFR = G::NFR;
  constexpr int NF = MODE == 1 ? BF / 2 : BF;         // output features per workgroup
  constexpr unsigned STAGE = G::STAGE;
  extern __shared__ __align__(16) unsigned char gm_smem[];   // NS stages of (weights BF rows, activations BT rows)
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wf = w % G::WFN, wt = w / G::WFN;
  // ---- tile of this workgroup
  int o = (int)(blockIdx.x & 7) * share + (int)(blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= share || o >= mt * nt * ksplit) return;
  const int slice = o / (mt * nt);                    // MODE 3: K slice of this workgroup (slices outermost)
  o -= slice * (mt * nt);
  const int kbeg = slice * (K / ksplit);
  const int per_panel = mt * GM_PANEL;
  const int panel = o / per_panel, in_panel = o - panel * per_panel;
  const int pw = min(GM_PANEL, nt - panel * GM_PANEL);        // the last panel may be narrower
  const int bt = in_panel / pw, bf = panel * GM_PANEL + in_panel % pw;
  const int m0 = bt * BT, n0 = bf * NF;
  // ---- fills: the XOR of the layout is applied on the global side: the lane that owns slot s (row s / CPR, physical
  // chunk s % CPR) fetches the logical chunk that belongs there.  Addresses are a per-workgroup buffer descriptor (the
  // tile's first row, its valid rows as the range), a per-lane byte offset and the k tile as the scalar offset.
  const int wv = __builtin_amdgcn_readfirstlane(w);   // wave-uniform by construction; keeps descriptors and LDS bases scalar
  const int rows_w = min(NF, N - n0), rows_a = min(BT, M - m0);
  const rsrc_t rs_w = make_rsrc(W + (size_t)n0 * K, (size_t)rows_w * K * 2);
  const rsrc_t rs_w2 = make_rsrc(MODE == 1 ? W2 + (size_t)n0 * K : W, MODE == 1 ? (size_t)rows_w * K * 2 : 0);
  const rsrc_t rs_a = make_rsrc(A + (size_t)m0 * lda, ((size_t)(rows_a - 1) * lda + K) * 2);
  unsigned wvoff[WL], avoff[AL];
#pragma unroll
  for (int j = 0; j < WL; ++j) {
    const int slot = (wv * WL + j) * 64 + lane, row = slot / G::CPR;
    const int ch = (int)((G::swz(row, slot % G::CPR) - (unsigned)row * G::RB) >> 4);   // XOR is its own inverse
    int n = row;
    if (MODE == 1) {
      // LDS rows of wave column wf': gate rows first, then the up rows of the same features (a fill instruction
      // covers 64 / CPR whole rows, all of them gate or all of them up)
      constexpr int HALF = 16 * FI;
      n = (row / (2 * HALF)) * HALF + (row % HALF);
    }
    wvoff[j] = (unsigned)n * (unsigned)K * 2u + (unsigned)ch * 16u;
  }
#pragma unroll
  for (int j = 0; j < AL; ++j) {
    const int slot = (wv * AL + j) * 64 + lane, row = slot / G::CPR;
    const int ch = (int)((G::swz(row, slot % G::CPR) - (unsigned)row * G::RB) >> 4);
    avoff[j] = (unsigned)row * (unsigned)lda * 2u + (unsigned)ch * 16u;
  }
  const unsigned wslot = (unsigned)(wv * WL) * 1024u, aslot = (unsigned)BF * G::RB + (unsigned)(wv * AL) * 1024u;
#define GM_FETCH(stage_, k0)                                                                                 \
  {                                                                                                          \
    unsigned char* st_ = gm_smem + (unsigned)(stage_) * STAGE;                                               \
    const unsigned so_ = (unsigned)(kbeg + (k0)) * 2u;                                                       \
    _Pragma("unroll") for (int j = 0; j < WL; ++j) {                                                         \
      const bool up_ = MODE == 1 && (((wv * WL + j) * (64 / G::CPR)) % (32 * FI)) >= 16 * FI;                \
      buf_load16_to_lds(up_ ? rs_w2 : rs_w, wvoff[j], so_, st_ + wslot + j * 1024);                          \
    }                                                                                                        \
    _Pragma("unroll") for (int j = 0; j < AL; ++j) buf_load16_to_lds(rs_a, avoff[j], so_, st_ + aslot + j * 1024); \
  }
#define GM_MFMAS(f_)                                                                                         \
  _Pragma("unroll") for (int i = 0; i < FI; ++i)                                                             \
    _Pragma("unroll") for (int j = 0; j < TJ; ++j)                                                           \
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f_[i]),               \
                                                          __builtin_bit_cast(bf16x8_t, f_[FI + j]), acc[i][j], 0, 0, 0);
  const int l32 = lane & 31, lh = lane >> 5;
  // fragment addresses inside a stage for the k steps of a tile (rows 32 apart share the XOR term)
  unsigned fw_off[KK], fa_off[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    fw_off[kk] = G::swz(wf * (32 * FI) + l32, kk * 2 + lh);
    fa_off[kk] = (unsigned)BF * G::RB + G::swz(wt * (32 * TJ) + l32, kk * 2 + lh);
  }
  floatx16_t acc[FI][TJ];
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  const int nkt = K / ksplit / G::BK;
  // Software pipeline over the k tiles.  NS-1 tiles are in flight ahead of the one being multiplied.  Within a tile the
  // fragments of k step kk+1 are read while step kk is multiplied; before the last step of tile kt the wave makes sure
  // its reads of the tile are complete, waits for its share of tile kt+1, meets the barrier (every wave's share has
  // landed, every wave has left the stage of tile kt), refills that stage with tile kt+NS and reads the first
  // fragments of tile kt+1 — so the MFMAs of the last step cover the barrier and those reads.  The compiler's own
  // schedule would wait for each fragment read in turn; the fences keep the order written here.
  constexpr int LPT = WL + AL;                        // fills per wave and tile
#pragma unroll
  for (int t = 0; t < NS - 1; ++t)
    if (t < nkt) GM_FETCH(t, t * G::BK)
  const unsigned smem0 = lds_addr(gm_smem);
  if (NS - 2 < nkt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPT) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();   // bare: the fence of __syncthreads would wait for the tiles still in flight
  if (NS - 1 < nkt) GM_FETCH(NS - 1, (NS - 1) * G::BK)
  u32x4_t fa_[NFR], fb_[NFR];                         // the two fragment sets, used by alternate k steps
  lds_read_rows<FI, 32 * G::RB>(fa_, smem0 + fw_off[0]);
  lds_read_rows<TJ, 32 * G::RB>(fa_ + FI, smem0 + fa_off[0]);
  int cur = 0;                                        // stage of tile kt
  for (int kt = 0; kt < nkt; ++kt) {
    const unsigned cb = smem0 + (unsigned)cur * STAGE;
    const int nxt = cur + 1 == NS ? 0 : cur + 1;
    __builtin_amdgcn_sched_barrier(0);
    lds_read_rows<FI, 32 * G::RB>(fb_, cb + fw_off[1]);
    lds_read_rows<TJ, 32 * G::RB>(fb_ + FI, cb + fa_off[1]);
    lds_wait<NFR>(fa_);
    GM_MFMAS(fa_)
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (KK == 4) {
      lds_read_rows<FI, 32 * G::RB>(fa_, cb + fw_off[2]);
      lds_read_rows<TJ, 32 * G::RB>(fa_ + FI, cb + fa_off[2]);
      lds_wait<NFR>(fb_);
      GM_MFMAS(fb_)
      __builtin_amdgcn_sched_barrier(0);
      lds_read_rows<FI, 32 * G::RB>(fb_, cb + fw_off[3]);
      lds_read_rows<TJ, 32 * G::RB>(fb_ + FI, cb + fa_off[3]);
      lds_wait<NFR>(fa_);
      GM_MFMAS(fa_)
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_wait<0>(fb_);                                 // this wave has left the stage of tile kt
    if (kt + 1 < nkt) {
      if (kt + NS - 1 < nkt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPT) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      if (kt + NS < nkt) GM_FETCH(cur, (kt + NS) * G::BK)
      const unsigned nb = smem0 + (unsigned)nxt * STAGE;
      lds_read_rows<FI, 32 * G::RB>(fa_, nb + fw_off[0]);
      lds_read_rows<TJ, 32 * G::RB>(fa_ + FI, nb + fa_off[0]);
    }
    __builtin_amdgcn_sched_barrier(0);
    GM_MFMAS(fb_)
    cur = nxt;
  }
#undef GM_FETCH
#undef GM_MFMAS
  // ---- epilogue.  D of a 32x32 tile: lane l holds row (token) l % 32 and features 8*(e/4) + 4*(l/32) + e%4
#pragma unroll
  for (int j = 0; j < TJ; ++j) {
    const int m = m0 + wt * (32 * TJ) + j * 32 + l32;
    if (m >= M) continue;
    if (MODE == 1) {
#pragma unroll
      for (int i = 0; i < FI / 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int f = n0 + wf * (16 * FI) + i * 32 + q * 8 + lh * 4;
          if (f >= N) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[e] = rnd_bf16(gelu_tanh_fast(rnd_bf16(acc[i][j][q * 4 + e]))) * rnd_bf16(acc[i + FI / 2][j][q * 4 + e]);
          *(uint2*)(C + (size_t)m * ldc + f) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
        }
    } else {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int f = n0 + wf * (32 * FI) + i * 32 + q * 8 + lh * 4;
          if (f >= N) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e];
          if (MODE == 3) {
            *(float4*)((float*)C + ((size_t)slice * M + m) * ldc + f) = make_float4(v[0], v[1], v[2], v[3]);
            continue;
          }
          if (MODE == 2) {
            const uint2 rv = *(const uint2*)(R + (size_t)m * ldr + f);
            v[0] = __uint_as_float(rv.x << 16) + rnd_bf16(v[0]);
            v[1] = __uint_as_float(rv.x & 0xffff0000u) + rnd_bf16(v[1]);
            v[2] = __uint_as_float(rv.y << 16) + rnd_bf16(v[2]);
            v[3] = __uint_as_float(rv.y & 0xffff0000u) + rnd_bf16(v[3]);
          }
          *(uint2*)(C + (size_t)m * ldc + f) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
        }
    }
  }
}

template <class G, int MODE>
int gemm_launch_tile(const void* A, long long lda, const void* W, const void* W2, const void* R, long long ldr, void* C,
                     long long ldc, int M, int N, int K, hipStream_t s, int ksplit = 1) {
  constexpr int NF = MODE == 1 ? G::BF / 2 : G::BF;
  static hipError_t attr_err = hipFuncSetAttribute((const void*)gemm_bf16_kernel<G, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS);
  if (attr_err != hipSuccess) { fstu_set_error("fstu_gemm_bf16: hipFuncSetAttribute: %s", hipGetErrorString(attr_err)); return (int)attr_err; }
  const int mt = (M + G::BT - 1) / G::BT, nt = (N + NF - 1) / NF;
  const long long tiles = (long long)mt * nt * ksplit;
  const int share = (int)((tiles + 7) / 8);
  hipLaunchKernelGGL((gemm_bf16_kernel<G, MODE>), dim3((unsigned)share * 8u), dim3(G::THREADS), G::LDS, s, (const bf16_t*)A, lda,
                     (const bf16_t*)W, (const bf16_t*)W2, (const bf16_t*)R, ldr, (bf16_t*)C, ldc, M, N, K, mt, nt, share, ksplit);
  return 0;
}

// ---------------------------------------------------------------- transposed activations
// C[b][m, n] = sum_k A[b][k, m] W[n, k]: the activations come as a slab with the REDUCTION index slowest (k rows of
// lda elements, m contiguous) — the time-major U+- of the exact-mode STU operator (flash_stu/modules/stu.py:107-120:
// tensordot of U (B, L, K, d) with M_phi (K, d, d) over (K, d); the filter-bank kernel writes U as (B, K*d, L) so
// that its stores are whole lines).  Same tiles, pipeline and epilogues as gemm_bf16_kernel (mode 0 and 2); what
// differs is the activation tile: LDS rows are k (BK rows of BT*2 bytes, filled 16 bytes = 8 consecutive m per lane),
// and the MFMA B fragment — 8 consecutive k of one m per lane — is gathered by two transposing reads
// (ds_read_b64_tr_b16: in a block of 16 lanes, lane i supplies the address of 4 consecutive m of row i/4 starting at
// column 4*(i%4), and receives column i of the 4 rows).  The 64-byte column groups of a row are XOR-ed with the row's
// low two bits, so the four rows of a read fall into different banks.  `nbatch` slabs run as one grid.
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ __forceinline__ u32x2_t lds_read_tr8(unsigned addr) {
  u32x2_t v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int N, int STEP, int I = 0>
__device__ __forceinline__ void lds_read_tr_cols(u32x2_t* f, const unsigned* addr) {   // N column tiles, rows k..k+3 and k+4..k+7
  if constexpr (I < N) {
    f[2 * I] = lds_read_tr8<0>(addr[I]);
    f[2 * I + 1] = lds_read_tr8<4 * STEP>(addr[I]);
    lds_read_tr_cols<N, STEP, I + 1>(f, addr);
  }
}
template <int LEFT>
__device__ __forceinline__ void lds_wait_n() { asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(LEFT)); }
template <int N> __device__ __forceinline__ void pin4(u32x4_t* f) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i]));
}
template <int N> __device__ __forceinline__ void pin2(u32x2_t* f) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i]));
}

template <class G, int MODE>
__global__ void __launch_bounds__(G::THREADS)
gemm_ta_bf16_kernel(const bf16_t* __restrict__ A, long long lda, long long sa, const bf16_t* __restrict__ W,
                    const bf16_t* __restrict__ R, long long ldr, long long sr, bf16_t* __restrict__ C, long long ldc,
                    long long sc, int M, int N, int K, int mt, int nt, int share, int nbatch) {
  constexpr int FI = G::FI, TJ = G::TJ, BF = G::BF, BT = G::BT, WL = G::WL, AL = G::AL, NS = G::NS, KK = G::KK;
  constexpr unsigned STAGE = G::STAGE;
  constexpr int RBT = BT * 2, CPRT = BT / 8;              // bytes and 16-byte chunks of an activation row (one k)
  constexpr int NRD = FI + 2 * TJ;                        // LDS reads per k step
  static_assert(G::BK == 64 && BT >= 128, "k tile of 64, at least 128 columns");
  static_assert((MODE == 0 || MODE == 2), "plain or residual epilogue");
  extern __shared__ __align__(16) unsigned char gm_smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wf = w % G::WFN, wt = w / G::WFN;
  int o = (int)(blockIdx.x & 7) * share + (int)(blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= share || o >= mt * nt * nbatch) return;
  const int batch = o / (mt * nt);
  o -= batch * (mt * nt);
  const int per_panel = mt * GM_PANEL;
  const int panel = o / per_panel, in_panel = o - panel * per_panel;
  const int pw = min(GM_PANEL, nt - panel * GM_PANEL);
  const int bt = in_panel / pw, bf = panel * GM_PANEL + in_panel % pw;
  const int m0 = bt * BT, n0 = bf * BF;
  A += (size_t)batch * sa;
  C += (size_t)batch * sc;
  if (MODE == 2) R += (size_t)batch * sr;
  const int wv = __builtin_amdgcn_readfirstlane(w);
  const int rows_w = min(BF, N - n0);
  const rsrc_t rs_w = make_rsrc(W + (size_t)n0 * K, (size_t)rows_w * K * 2);
  const rsrc_t rs_a = make_rsrc(A + m0, ((size_t)(K - 1) * lda + BT) * 2);     // M % BT == 0: whole rows of BT columns
  unsigned wvoff[WL], avoff[AL];
#pragma unroll
  for (int j = 0; j < WL; ++j) {
    const int slot = (wv * WL + j) * 64 + lane, row = slot / G::CPR;
    const int ch = (int)((G::swz(row, slot % G::CPR) - (unsigned)row * G::RB) >> 4);
    wvoff[j] = (unsigned)row * (unsigned)K * 2u + (unsigned)ch * 16u;
  }
#pragma unroll
  for (int j = 0; j < AL; ++j) {
    const int slot = (wv * AL + j) * 64 + lane, kr = slot / CPRT, pc = slot % CPRT;
    const int lc = pc ^ (4 * (kr & 3));                  // the XOR is its own inverse
    avoff[j] = (unsigned)kr * (unsigned)lda * 2u + (unsigned)lc * 16u;
  }
  const unsigned wslot = (unsigned)(wv * WL) * 1024u, aslot = (unsigned)BF * G::RB + (unsigned)(wv * AL) * 1024u;
#define GT_FETCH(stage_, k0)                                                                                 \
  {                                                                                                          \
    unsigned char* st_ = gm_smem + (unsigned)(stage_) * STAGE;                                               \
    const unsigned sw_ = (unsigned)(k0) * 2u;                                                                \
    const unsigned sa_ = (unsigned)((size_t)(k0) * (size_t)lda * 2u);                                        \
    _Pragma("unroll") for (int j = 0; j < WL; ++j) buf_load16_to_lds(rs_w, wvoff[j], sw_, st_ + wslot + j * 1024); \
    _Pragma("unroll") for (int j = 0; j < AL; ++j) buf_load16_to_lds(rs_a, avoff[j], sa_, st_ + aslot + j * 1024); \
  }
  struct Frag8 { u32x2_t lo, hi; };
#define GT_MFMAS(fw_, fx_)                                                                                   \
  _Pragma("unroll") for (int i = 0; i < FI; ++i)                                                             \
    _Pragma("unroll") for (int j = 0; j < TJ; ++j) {                                                         \
      const Frag8 b_ = {fx_[2 * j], fx_[2 * j + 1]};                                                         \
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fw_[i]),              \
                                                          __builtin_bit_cast(bf16x8_t, b_), acc[i][j], 0, 0, 0); \
    }
  const int l32 = lane & 31, lh = lane >> 5;
  unsigned fw_off[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) fw_off[kk] = G::swz(wf * (32 * FI) + l32, kk * 2 + lh);
  // transposing reads: this lane's address inside a stage for column tile j at k step 0, rows k..k+3
  const int blk = lane >> 4, i16 = lane & 15, key = i16 >> 2;
  unsigned ta_off[TJ];
#pragma unroll
  for (int j = 0; j < TJ; ++j)
    ta_off[j] = (unsigned)BF * G::RB + (unsigned)(8 * (blk >> 1) + key) * RBT + (unsigned)(((wt * TJ + j) ^ key) << 6) +
                (unsigned)(2 * (blk & 1) + ((i16 & 3) >> 1)) * 16u + (unsigned)(i16 & 1) * 8u;
  floatx16_t acc[FI][TJ];
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  const int nkt = K / G::BK;
  constexpr int LPT = WL + AL;
#pragma unroll
  for (int t = 0; t < NS - 1; ++t)
    if (t < nkt) GT_FETCH(t, t * G::BK)
  const unsigned smem0 = lds_addr(gm_smem);
  if (NS - 2 < nkt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPT) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  if (NS - 1 < nkt) GT_FETCH(NS - 1, (NS - 1) * G::BK)
  u32x4_t wa_[FI], wb_[FI];                           // weight fragments of alternate k steps
  u32x2_t xa_[2 * TJ], xb_[2 * TJ];                   // activation fragments (two halves per column tile)
  unsigned ta[TJ];
#define GT_READ(fw_, fx_, base_, kk_)                                                                        \
  {                                                                                                          \
    lds_read_rows<FI, 32 * G::RB>(fw_, (base_) + fw_off[kk_]);                                               \
    _Pragma("unroll") for (int j = 0; j < TJ; ++j) ta[j] = (base_) + ta_off[j] + (unsigned)(kk_) * 16u * RBT; \
    lds_read_tr_cols<TJ, RBT>(fx_, ta);                                                                      \
  }
#define GT_WAIT(left_, fw_, fx_)                                                                             \
  {                                                                                                          \
    lds_wait_n<left_>();                                                                                     \
    pin4<FI>(fw_);                                                                                           \
    pin2<2 * TJ>(fx_);                                                                                       \
  }
  GT_READ(wa_, xa_, smem0, 0)
  int cur = 0;
  for (int kt = 0; kt < nkt; ++kt) {
    const unsigned cb = smem0 + (unsigned)cur * STAGE;
    const int nxt = cur + 1 == NS ? 0 : cur + 1;
    __builtin_amdgcn_sched_barrier(0);
    GT_READ(wb_, xb_, cb, 1)
    GT_WAIT(NRD, wa_, xa_)
    GT_MFMAS(wa_, xa_)
    __builtin_amdgcn_sched_barrier(0);
    GT_READ(wa_, xa_, cb, 2)
    GT_WAIT(NRD, wb_, xb_)
    GT_MFMAS(wb_, xb_)
    __builtin_amdgcn_sched_barrier(0);
    GT_READ(wb_, xb_, cb, 3)
    GT_WAIT(NRD, wa_, xa_)
    GT_MFMAS(wa_, xa_)
    __builtin_amdgcn_sched_barrier(0);
    GT_WAIT(0, wb_, xb_)                              // this wave has left the stage of tile kt
    if (kt + 1 < nkt) {
      if (kt + NS - 1 < nkt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPT) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      if (kt + NS < nkt) GT_FETCH(cur, (kt + NS) * G::BK)
      const unsigned nb = smem0 + (unsigned)nxt * STAGE;
      GT_READ(wa_, xa_, nb, 0)
    }
    __builtin_amdgcn_sched_barrier(0);
    GT_MFMAS(wb_, xb_)
    cur = nxt;
  }
#undef GT_FETCH
#undef GT_MFMAS
#undef GT_READ
#undef GT_WAIT
  // ---- epilogue: lane l holds row (position) l % 32 and features 8*(e/4) + 4*(l/32) + e%4 of a 32x32 tile
#pragma unroll
  for (int j = 0; j < TJ; ++j) {
    const int m = m0 + wt * (32 * TJ) + j * 32 + l32;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < FI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int f = n0 + wf * (32 * FI) + i * 32 + q * 8 + lh * 4;
        if (f >= N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e];
        if (MODE == 2) {
          const uint2 rv = *(const uint2*)(R + (size_t)m * ldr + f);
          v[0] = __uint_as_float(rv.x << 16) + rnd_bf16(v[0]);
          v[1] = __uint_as_float(rv.x & 0xffff0000u) + rnd_bf16(v[1]);
          v[2] = __uint_as_float(rv.y << 16) + rnd_bf16(v[2]);
          v[3] = __uint_as_float(rv.y & 0xffff0000u) + rnd_bf16(v[3]);
        }
        *(uint2*)(C + (size_t)m * ldc + f) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
      }
  }
}

template <class G, int MODE>
int gemm_ta_launch_tile(const void* A, long long lda, long long sa, const void* W, const void* R, long long ldr, long long sr,
                        void* C, long long ldc, long long sc, int M, int N, int K, int nbatch, hipStream_t s) {
  static hipError_t attr_err = hipFuncSetAttribute((const void*)gemm_ta_bf16_kernel<G, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS);
  if (attr_err != hipSuccess) { fstu_set_error("fstu_gemm_bf16_ta: hipFuncSetAttribute: %s", hipGetErrorString(attr_err)); return (int)attr_err; }
  const int mt = M / G::BT, nt = (N + G::BF - 1) / G::BF;
  const long long tiles = (long long)mt * nt * nbatch;
  const int share = (int)((tiles + 7) / 8);
  hipLaunchKernelGGL((gemm_ta_bf16_kernel<G, MODE>), dim3((unsigned)share * 8u), dim3(G::THREADS), G::LDS, s, (const bf16_t*)A, lda, sa,
                     (const bf16_t*)W, (const bf16_t*)R, ldr, sr, (bf16_t*)C, ldc, sc, M, N, K, mt, nt, share, nbatch);
  return 0;
}

int gemm_cus() {
  static int cus = [] {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return 256;
    return p.multiProcessorCount;
  }();
  return cus;
}

//                     waves  tiles  BK  stages
using TileBig = GemmTile<4, 2, 2, 4, 64, 2>;     // 256 x 256, 8 waves, 128 KB of LDS
using TileSmall = GemmTile<2, 2, 2, 2, 64, 2>;   // 128 x 128, 4 waves, 64 KB: two workgroups per compute unit
using TileDeep = GemmTile<2, 2, 2, 2, 64, 4>;    // 128 x 128, 4 waves, 3 tiles in flight: one workgroup per compute unit
using TileRows32 = GemmTile<2, 1, 2, 1, 64, 4>;  // 128 features x 32 rows, 2 waves, 80 KB: weight streaming, two workgroups per compute unit
using Tile96 = GemmTile<1, 4, 3, 1, 64, 4>;      // 96 features x 128 rows, 4 waves, 112 KB: N = 768 or 2304 in whole tiles
using TileK32 = GemmTile<2, 2, 4, 2, 32, 3>;     // 256 x 128, 4 waves, 72 KB, k tiles of 32 for K % 64 != 0

template <int MODE>
int gemm_launch(const void* A, long long lda, const void* W, const void* W2, const void* R, long long ldr, void* C, long long ldc,
                int M, int N, int K, hipStream_t s) {
  if (K % 64 != 0) return gemm_launch_tile<TileK32, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
  if (M <= 32) return gemm_launch_tile<TileRows32, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
  // Measured choices (MI355X, bf16): the large tile halves the fill traffic per flop and pays once K amortises its
  // start-up and the grid still covers the chip twice (M=32768, K >= 2048: 1.01-1.18 PFLOP/s against 0.89-0.99;
  // M=4096, N=9216, K=768: 92 us against 80 us).  A grid that leaves one workgroup per compute unit anyway gains from
  // the deeper pipeline when K is long (M=4096, N=768, K=9216: 83 us against 93 us).
  const int nf = MODE == 1 ? 2 : 1;
  const long long big = (long long)((M + 255) / 256) * ((N * nf + 255) / 256);
  const long long small = (long long)((M + 127) / 128) * ((N * nf + 127) / 128);
  if (K >= 1024 && big >= 2 * gemm_cus()) return gemm_launch_tile<TileBig, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
  if constexpr (MODE != 1) {
    // A feature count that is a whole number of 96-wide tiles but leaves compute units idle (or nearly idle in a last
    // round) with 128-wide ones: the time follows the rounds a compute unit runs times the area of a tile
    // (N = 768, M = 4096: 192 tiles of 128 x 128 on 256 CUs against 256 tiles of 96 x 128).  Only where the 128-wide
    // grid does not fill the chip: with several rounds per compute unit two resident workgroups of 128 x 128 cover
    // each other's start and end (N = 2304, M = 4096: 28.5 us against 35.2 us for the 96-wide tile).
    const long long cus = gemm_cus(), t96 = (long long)((M + 127) / 128) * (N / 96);
    if (N % 96 == 0 && small <= cus && ((t96 + cus - 1) / cus) * 96 < ((small + cus - 1) / cus) * 128)
      return gemm_launch_tile<Tile96, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
  }
  if (K >= 2048 && small <= gemm_cus()) return gemm_launch_tile<TileDeep, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
  return gemm_launch_tile<TileSmall, MODE>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, s);
}

}  // namespace

extern "C" int fstu_gemm_bf16_splitk(const void* A, int64_t lda, const void* W, float* partial, int M, int N, int K, int ksplit,
                                     void* stream) {
  FSTU_REQUIRE(A && W && partial, FSTU_ENULL, "fstu_gemm_bf16_splitk: null pointer");
  FSTU_REQUIRE(ksplit >= 1 && ksplit <= 64 && K % (64 * ksplit) == 0, FSTU_ESHAPE,
               "fstu_gemm_bf16_splitk: K=%d must be a multiple of 64*ksplit (ksplit=%d, 1..64)", K, ksplit);
  FSTU_REQUIRE(M >= 1 && N >= 4 && N % 4 == 0 && lda >= K && lda % 8 == 0, FSTU_ESHAPE,
               "fstu_gemm_bf16_splitk: M=%d N=%d (N %% 4 == 0) lda=%lld", M, N, (long long)lda);
  FSTU_REQUIRE(fstu_aligned(A, 16) && fstu_aligned(W, 16) && fstu_aligned(partial, 16), FSTU_EALIGN,
               "fstu_gemm_bf16_splitk: pointers must be 16-byte aligned");
  FSTU_REQUIRE(lda < GM_MAX_LD && K < GM_MAX_LD, FSTU_ESHAPE, "fstu_gemm_bf16_splitk: lda=%lld / K=%d beyond the 32-bit tile offsets",
               (long long)lda, K);
  int rc;
  if (M <= 32) rc = gemm_launch_tile<TileRows32, 3>(A, lda, W, nullptr, nullptr, 0, partial, N, M, N, K, (hipStream_t)stream, ksplit);
  else rc = gemm_launch_tile<TileSmall, 3>(A, lda, W, nullptr, nullptr, 0, partial, N, M, N, K, (hipStream_t)stream, ksplit);
  if (rc) return rc;
  FSTU_CHECK_LAUNCH("fstu_gemm_bf16_splitk");
  return FSTU_OK;
}

extern "C" int fstu_gemm_bf16(const void* A, int64_t lda, const void* W, const void* W2, const void* R, int64_t ldr, void* C,
                              int64_t ldc, int M, int N, int K, int mode, void* stream) {
  FSTU_REQUIRE(A && W && C, FSTU_ENULL, "fstu_gemm_bf16: null pointer");
  FSTU_REQUIRE(mode >= 0 && mode <= 2, FSTU_EARG, "fstu_gemm_bf16: mode %d", mode);
  FSTU_REQUIRE((mode != 1 || W2) && (mode != 2 || R), FSTU_ENULL, "fstu_gemm_bf16: mode %d needs its second operand", mode);
  FSTU_REQUIRE(M >= 1 && N >= 4 && N % 4 == 0 && K >= 32 && K % 32 == 0, FSTU_ESHAPE,
               "fstu_gemm_bf16: need K %% 32 == 0 and N %% 4 == 0 (M=%d N=%d K=%d)", M, N, K);
  FSTU_REQUIRE(lda >= K && lda % 8 == 0 && ldc >= N && ldc % 4 == 0 && (mode != 2 || (ldr >= N && ldr % 4 == 0)), FSTU_ESHAPE,
               "fstu_gemm_bf16: row strides (lda=%lld ldc=%lld ldr=%lld)", (long long)lda, (long long)ldc, (long long)ldr);
  FSTU_REQUIRE(fstu_aligned(A, 16) && fstu_aligned(W, 16) && fstu_aligned(W2, 16) && fstu_aligned(C, 8) && fstu_aligned(R, 8),
               FSTU_EALIGN, "fstu_gemm_bf16: pointers must be 16-byte aligned (C, R: 8)");
  FSTU_REQUIRE(lda < GM_MAX_LD && K < GM_MAX_LD, FSTU_ESHAPE, "fstu_gemm_bf16: lda=%lld / K=%d beyond the 32-bit tile offsets",
               (long long)lda, K);
  int rc;
  if (mode == 0) rc = gemm_launch<0>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, (hipStream_t)stream);
  else if (mode == 1) rc = gemm_launch<1>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, (hipStream_t)stream);
  else rc = gemm_launch<2>(A, lda, W, W2, R, ldr, C, ldc, M, N, K, (hipStream_t)stream);
  if (rc) return rc;
  FSTU_CHECK_LAUNCH("fstu_gemm_bf16");
  return FSTU_OK;
}

// C[b] = T(A[b]^T W^T) (mode 0) or T(R[b] + T(A[b]^T W^T)) (mode 2) for nbatch slabs A[b] of shape (K, M) with row
// stride lda (elements; the reduction index slowest, M contiguous), W (N, K) row-major.  M must be a multiple of 128.
extern "C" int fstu_gemm_bf16_ta(const void* A, int64_t lda, int64_t batch_stride_a, const void* W, const void* R, int64_t ldr,
                                 int64_t batch_stride_r, void* C, int64_t ldc, int64_t batch_stride_c, int M, int N, int K,
                                 int nbatch, int mode, void* stream) {
  FSTU_REQUIRE(A && W && C, FSTU_ENULL, "fstu_gemm_bf16_ta: null pointer");
  FSTU_REQUIRE(mode == 0 || mode == 2, FSTU_EARG, "fstu_gemm_bf16_ta: mode %d (0: plain, 2: residual add)", mode);
  FSTU_REQUIRE(mode != 2 || R, FSTU_ENULL, "fstu_gemm_bf16_ta: mode 2 needs R");
  FSTU_REQUIRE(M >= 128 && M % 128 == 0 && N >= 4 && N % 4 == 0 && K >= 64 && K % 64 == 0 && nbatch >= 1, FSTU_ESHAPE,
               "fstu_gemm_bf16_ta: need M %% 128 == 0, N %% 4 == 0, K %% 64 == 0 (M=%d N=%d K=%d nbatch=%d)", M, N, K, nbatch);
  FSTU_REQUIRE(lda >= M && lda % 8 == 0 && ldc >= N && ldc % 4 == 0 && (mode != 2 || (ldr >= N && ldr % 4 == 0)), FSTU_ESHAPE,
               "fstu_gemm_bf16_ta: row strides (lda=%lld ldc=%lld ldr=%lld)", (long long)lda, (long long)ldc, (long long)ldr);
  // 32-bit byte offsets inside a slab (buffer addressing) and inside W
  FSTU_REQUIRE((unsigned long long)K * (unsigned long long)lda * 2ull < 0xfff00000ull && (unsigned long long)N * K * 2ull < 0xfff00000ull,
               FSTU_ESHAPE, "fstu_gemm_bf16_ta: a slab (K*lda) or W (N*K) exceeds 4 GB of 32-bit offsets");
  FSTU_REQUIRE(lda < GM_MAX_LD && K < GM_MAX_LD, FSTU_ESHAPE, "fstu_gemm_bf16_ta: lda=%lld / K=%d beyond the 32-bit tile offsets",
               (long long)lda, K);
  FSTU_REQUIRE(batch_stride_a % 8 == 0 && batch_stride_c % 4 == 0 && batch_stride_r % 4 == 0, FSTU_ESHAPE,
               "fstu_gemm_bf16_ta: batch strides must keep the alignment");
  FSTU_REQUIRE(fstu_aligned(A, 16) && fstu_aligned(W, 16) && fstu_aligned(C, 8) && fstu_aligned(R, 8), FSTU_EALIGN,
               "fstu_gemm_bf16_ta: pointers must be 16-byte aligned (C, R: 8)");
  hipStream_t s = (hipStream_t)stream;
  const long long big = (long long)(M / 256) * ((N + 255) / 256) * nbatch;
  int rc;
#define TA_GO(TILE)                                                                                                              \
  (mode == 0 ? gemm_ta_launch_tile<TILE, 0>(A, lda, batch_stride_a, W, R, ldr, batch_stride_r, C, ldc, batch_stride_c, M, N, K,  \
                                            nbatch, s)                                                                           \
             : gemm_ta_launch_tile<TILE, 2>(A, lda, batch_stride_a, W, R, ldr, batch_stride_r, C, ldc, batch_stride_c, M, N, K,  \
                                            nbatch, s))
  if (M % 256 == 0 && K >= 1024 && big >= 2 * gemm_cus()) rc = TA_GO(TileBig);
  else rc = TA_GO(TileSmall);
#undef TA_GO
  if (rc) return rc;
  FSTU_CHECK_LAUNCH("fstu_gemm_bf16_ta");
  return FSTU_OK;
}
