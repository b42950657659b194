/*
 * flashstu_hip.h -- C ABI of libflashstu_hip.so: hand-written gfx950 (MI355X)
 * kernels for Flash STU's autoregressive token loop.
 *
 * The reference (hazan-lab/flash-stu-2) has no native code of its own: every
 * device computation on this path is delegated to torch ops or third-party
 * CUDA/Triton wheels.  Each entry point below names the reference call site
 * (file:line, relative to the reference checkout) whose arithmetic it replaces.
 *
 * Conventions
 *   - All pointers are DEVICE pointers owned by the caller unless stated.
 *     The library allocates nothing.
 *   - `dtype` selects the model dtype of activations and weights:
 *     FSTU_F32 or FSTU_BF16.  Accumulation is always fp32; values are rounded
 *     to the model dtype (round-to-nearest-even) at the points where the
 *     reference's torch ops round.
 *   - All tensors are dense row-major; row strides are given where a tensor
 *     may be a view.
 *   - `stream` is a hipStream_t passed as void*.  Launches are asynchronous on
 *     that stream; no entry point synchronises.
 *   - Return value: 0 on success; negative FSTU_E* for rejected arguments
 *     (nothing is launched); positive values are hipError_t codes.
 *     fstu_last_error() returns a thread-local description of the last failure.
 */
#ifndef FLASHSTU_HIP_H
#define FLASHSTU_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSTU_VERSION 100

enum { FSTU_F32 = 0, FSTU_BF16 = 1 };

enum {
  FSTU_OK = 0,
  FSTU_ENULL = -1,   /* null pointer */
  FSTU_EDTYPE = -2,  /* unknown dtype */
  FSTU_ESHAPE = -3,  /* dimension out of the supported range */
  FSTU_EALIGN = -4,  /* pointer or stride not aligned as required */
  FSTU_EARG = -5     /* other invalid argument */
};

int fstu_version(void);
const char* fstu_last_error(void);

/* Maximum number of activation rows the skinny (decode) kernels accept. */
#define FSTU_MAX_DECODE_ROWS 16

/* ---- embedding ---------------------------------------------------------
 * out[r,:] = table[ids[r],:].   Replaces nn.Embedding at flash_stu/model.py:152.
 * ids are int64; an id outside [0,vocab) is rejected on the device by clamping
 * (the row of id clamp(id,0,vocab-1) is returned). */
int fstu_embed(const int64_t* ids, const void* table, void* out, int rows, int d, int vocab,
               int dtype, void* stream);

/* ---- RMSNorm with fused residual add -------------------------------------
 * Optional residual update followed by optional RMSNorm:
 *   if delta != NULL:  x[r,:] = T( x[r,:] + D[r,:] )   (in place)
 *   if y != NULL:      y[r,:] = T( x[r,:] * rsqrt(mean(x[r,:]^2)+eps) * w )
 * D depends on delta_mode:
 *   0: delta is (rows,d) in the model dtype.
 *   1: delta is `nslices` fp32 slices (nslices,rows,d); D = T(sum of slices in
 *      slice order)  -- the split-K partial sums of fstu_linear_decode_splitk.
 *   2: delta is fp32 (nslices,2,rows,d) holding even-lag / odd-lag partial sums
 *      E,O of the STU convolution; D = T( T(E+O) + T(E-O) ) when both branches
 *      are used (single_branch==0) or T(E+O) otherwise
 *      (flash_stu/utils/stu_utils.py:226-228, modules/stu.py:120).
 * Replaces torch.nn.RMSNorm + x.add_() at flash_stu/layers/stu_layer.py:81,93,96,
 * layers/attention_layer.py:53-62, model.py:173. */
int fstu_add_rmsnorm(void* x, const void* delta, int delta_mode, int nslices, int single_branch,
                     const void* w, void* y, int rows, int d, float eps, int dtype, void* stream);
/* The residual update of delta_mode 1 alone, spread over the whole chip (4 elements per thread): x = T(x + T(sum of
 * the slices)), the same values as fstu_add_rmsnorm leaves in x; for a consumer that forms the norm itself
 * (fstu_linear_packed with norm_w at 17..32 rows).  The x.add_() of flash_stu/layers/stu_layer.py:96 and
 * layers/attention_layer.py:62 behind a split-K down projection.  bf16, d % 4 == 0. */
int fstu_add_slices(void* x, const float* slices, int nslices, int rows, int d, int dtype, void* stream);

/* ---- skinny linear layers for decode (rows <= 16) -------------------------
 * y[m, n] = T( sum_k x[m,k] * W[n,k] ),  W is (N,K) row-major (nn.Linear layout).
 * x rows have stride ldx elements, y rows stride ldy.  bf16 uses MFMA and needs
 * K % 64 == 0; other shapes and fp32 take a vector-ALU kernel.
 * Replaces nn.Linear / `@` at flash_stu/modules/attention.py:74,101,
 * modules/stu.py:87 (with M_inputs pre-transposed), model.py:176. */
int fstu_linear_decode(const void* x, int ldx, const void* W, void* y, int ldy, int rows, int N, int K,
                       int dtype, void* stream);

/* act[m,i] = T( T(gelu_tanh(T(x.Wg[i]))) * T(x.Wu[i]) ), Wg/Wu (I,K).
 * Replaces gate_proj/up_proj/gelu/mul at flash_stu/modules/swiglu.py:23-26. */
int fstu_glu_decode(const void* x, int ldx, const void* Wg, const void* Wu, void* act, int ldact, int rows,
                    int I, int K, int dtype, void* stream);

/* Split-K form: partial[s, m, n] = sum over the s-th K range of x[m,k] W[n,k]
 * (fp32, no rounding), s < ksplit.  The consumer (fstu_add_rmsnorm mode 1) adds
 * the slices in order, so results are deterministic.  K % (64*ksplit) == 0 for
 * bf16.  Replaces down_proj at flash_stu/modules/swiglu.py:27. */
int fstu_linear_decode_splitk(const void* x, int ldx, const void* W, float* partial, int rows, int N, int K,
                              int ksplit, int dtype, void* stream);

/* Elementwise act = T( T(gelu_tanh(g)) * u ) over n elements (prefill form of
 * flash_stu/modules/swiglu.py:24-26). */
int fstu_gelu_mul(const void* g, const void* u, void* act, int64_t n, int dtype, void* stream);

/* In place y[r,c] = act( T(y[r,c] + bias[c]) ) over (rows,n); bias may be NULL; kind 0: identity, 1: SiLU.
 * The `bias=True` linears (flash_stu/modules/swiglu.py:12-20, modules/attention.py:27-36) and the SiLU of the
 * STU sandwich (flash_stu/layers/stu_layer.py:49,84-85) on top of the bias-free GEMV kernels. */
int fstu_bias_act(void* y, const void* bias, int64_t rows, int n, int kind, int dtype, void* stream);

/* ---- STU decode step: exact history form ----------------------------------
 * hist is the (B,cap,d) history of projected inputs x_proj (model dtype), the
 * newest at time index t (0-based, t < cap); filt is the (L,d) per-channel
 * filter phi_proj in the model dtype.  Writes fp32 partial sums
 *   eo[s,0,b,c] = sum over even lags in lag range s of filt[lag,c]*hist[b,t-lag,c]
 *   eo[s,1,b,c] = same over odd lags
 * for nsplit lag ranges covering lags 0..min(t,L-1); consumed by
 * fstu_add_rmsnorm mode 2.  Restates convolve() at
 * flash_stu/utils/stu_utils.py:223-228 at the newest position. */
int fstu_stu_step_hist(const void* hist, const void* filt, float* eo, int B, int d, int t, int cap, int L,
                       int nsplit, int dtype, void* stream);

/* ---- STU decode step: distilled diagonal recurrence (LDS form) -------------
 * state is fp32 (B,2,S,d): two parity banks of S modes per (batch,channel).
 * The bank of parity t&1 is advanced h_j <- a[j]*h_j + xp[b,c] and
 *   y[b,c] = T( 2 * sum_j ce[j,c]*h_j )
 * where a (S) are the two-step poles and ce (S,d) the per-channel output
 * weights fitted to phi_proj's even lags.  Per-token form of
 * mini_stu/stu_lds.py:213-338 merged with the approx-mode contraction of
 * flash_stu/modules/stu.py:87-98,120. */
int fstu_stu_step_lds(float* state, const void* xp, int ldxp, const float* a, const float* ce, void* y, int ldy,
                      int B, int S, int d, int t, int dtype, void* stream);

/* The two-branch step with the reference's rounding points: besides E = sum_j ce[j,c]*h_j over the bank of parity t&1
 * (after its advance; even lags), O = sum_j co[j,c]*h_j over the other bank (odd lags: lag 2m+1 reaches position
 * t-1-2m), co (S,d) fitted to phi_proj's odd lags, and
 *   y[b,c] = T( T(E + O) + T(E - O) )
 * i.e. the plus and the minus branch rounded to the model dtype separately before their sum
 * (flash_stu/utils/stu_utils.py:226-228, flash_stu/modules/stu.py:120); fstu_stu_step_lds returns T(2E).
 *
 * Optional exact head of the filter (ring, fir, fir_taps all given, or NULL / NULL / 0): the recurrence reproduces
 * phi_proj (flash_stu/modules/stu.py:88) only up to its lag-by-lag rounding to the model dtype, which is largest on the
 * first lags.  fir (fir_taps,d) fp32 holds phi_proj[s,c] minus the fitted filter for the first fir_taps lags (a power of
 * two, 8..1024), ring (B,fir_taps,d) in the model dtype the last projected inputs (position p in slot p % fir_taps, zero
 * before the first position): the even lags' correction joins E, the odd lags' O, and the step stores xp in slot
 * t % fir_taps. */
int fstu_stu_step_lds_pair(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                           void* ring, const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int t,
                           int dtype, void* stream);
/* The pair step without the read of the other bank.  The odd-lag sum O of position t weighs the bank that the step at
 * t-1 advanced and the odd lags of the exact head reach inputs that step already held, so the step at t-1 can form it
 * while it has that bank in registers: ocache (B,d) fp32 holds the O of position t on entry and the O of position t+1
 * on return.  Same values as fstu_stu_step_lds_pair, bit for bit (same products in the same order), a third less state
 * traffic.  res: NULL, or the residual rows as in fstu_stu_step_lds_pair_add.  fstu_stu_step_lds_prime fills ocache for
 * position t+1 from the state and the ring as they stand after position t (a prompt's last position); it advances and
 * writes nothing else.  No counterpart in the reference, whose STU layers keep no decode state
 * (flash_stu/layers/stu_layer.py:99-120). */
int fstu_stu_step_lds_pair_cached(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                                  void* ring, const float* fir, int fir_taps, float* ocache, const void* res, void* y, int ldy,
                                  int B, int S, int d, int t, int dtype, void* stream);
int fstu_stu_step_lds_prime(const float* state, const float* a, const float* co, const void* ring, const float* fir,
                            int fir_taps, float* ocache, int B, int S, int d, int t, int dtype, void* stream);
/* The same step joining the residual stream (flash_stu/layers/stu_layer.py:93, x = x + stu(stu_norm(x))):
 * y = T(res + T(step output)), rows of stride ldy in both, 16-byte aligned; y may be res. */
int fstu_stu_step_lds_pair_add(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                               void* ring, const float* fir, int fir_taps, const void* res, void* y, int ldy, int B, int S,
                               int d, int t, int dtype, void* stream);

/* The same step for the single-branch filters of use_hankel_L=True (flash_stu/utils/stu_utils.py:22-25,229-246:
 * one convolution over ALL lags, no sign branch): ce (S,d) is fitted to the even lags and weighs the bank of parity
 * t&1 after its advance, co (S,d) is fitted to the odd lags and weighs the other bank (lag 2m+1 reaches position
 * t-1-2m):  y[b,c] = T( sum_j ce[j,c]*h_j[bank t&1] + sum_j co[j,c]*h_j[other bank] ). */
int fstu_stu_step_lds_single(float* state, const void* xp, int ldxp, const float* a, const float* ce, const float* co,
                             void* y, int ldy, int B, int S, int d, int t, int dtype, void* stream);

/* Exact mode (use_approx=False) on the same two-bank state, fed with the raw inputs x (B,d): after advancing the bank
 * of parity t&1,  E_k = sum_j ce[j,k] h_j[that bank],  O_k = sum_j co[j,k] h_j[other bank]  and
 *   u_plus[b,k,c] = T(E_k + O_k),  u_minus[b,k,c] = T(E_k - O_k)   (u_minus / co may be NULL: single branch)
 * with ce, co (S,K) fitted to the even / odd lags of the K filters.  Outputs are (B,K,d); the contraction with
 * M_phi_plus / M_phi_minus (flash_stu/modules/stu.py:107-120) follows as two skinny GEMVs.  K <= 32. */
int fstu_stu_bank_step_lds(float* state, const void* x, int ldx, const float* a, const float* ce, const float* co,
                           void* u_plus, void* u_minus, int B, int S, int d, int K, int t, int dtype, void* stream);

/* Input projection and recurrence step in one launch (bf16, K % 256 == 0):
 *   xp[b,c] = T( h[b,:] . Mt[c,:] )  with Mt = M_inputs^T (d,K) row-major, then the step of
 * fstu_stu_step_lds_pair on xp (co != NULL; ring / fir / fir_taps as there) or of fstu_stu_step_lds (co == NULL).
 * xp_out (B,d) receives xp when not NULL.
 * Replaces `x @ M_inputs` + the convolution at flash_stu/modules/stu.py:87-98,120 for one token. */
int fstu_stu_inproj_step(const void* h, int ldh, const void* Mt, float* state, const float* a, const float* ce,
                         const float* co, void* ring, const float* fir, int fir_taps, void* y, int ldy, void* xp_out, int B,
                         int S, int d, int K, int t, void* stream);

/* The same launch with the residual update and the RMSNorm of its input as the prologue
 * (flash_stu/layers/stu_layer.py:78-82 after the previous layer's :93-97): x' = T(x_in + T(sum of nslices <= 4 fp32
 * (B,K) slices)) goes to x_out (not x_in itself), h = rmsnorm(x') * norm_w feeds the projection.  K % 256 == 0,
 * B*K/8 <= 1024. */
int fstu_stu_res_inproj_step(const void* x_in, const float* slices, int nslices, void* x_out, const void* norm_w, float eps,
                             const void* Mt, float* state, const float* a, const float* ce, const float* co, void* ring,
                             const float* fir, int fir_taps, void* y, int ldy, int B, int S, int d, int K, int t, void* stream);

/* The step of fstu_stu_step_lds applied to T consecutive positions t_start .. t_start+T-1 in one launch (scan form
 * of the prefill: no FFT, no history buffer): y[b,t,c] for every position and the state after the last one.
 * xp, y are (B,T,d) with element strides (x_bstride, x_tstride, 1) / (y_bstride, y_tstride, 1), rows 16-byte aligned;
 * carry 0 starts from a zero state (state is output only), carry 1 continues from the state given.  S <= 128.
 * The final state equals T calls of fstu_stu_step_lds bit for bit; the outputs differ from theirs only by the order
 * of the sum over the S modes.  Sequence counterpart of the reference's scan, mini_stu/stu_lds.py:17-68 (Triton
 * lds_scan_kernel) and :279-338 (FixedDiagonalLDS.forward), merged with the approx-mode contraction of
 * flash_stu/modules/stu.py:87-98,120. */
int fstu_stu_scan_lds(const void* xp, int64_t x_bstride, int64_t x_tstride, const float* a, const float* ce,
                      float* state, void* y, int64_t y_bstride, int64_t y_tstride, int B, int T, int S, int d,
                      int t_start, int carry, int dtype, void* stream);

/* Builds that state from a prefilled history: for both parities p,
 *   state[b,p,j,c] = sum_{m>=0} a[j]^m * hist[b, tp-2m, c],  tp = newest index
 *   of parity p that is <= t_last.  hist is (B,cap,d). */
int fstu_stu_lds_state_from_hist(const void* hist, const float* a, float* state, int B, int S, int d,
                                 int t_last, int cap, int dtype, void* stream);
/* The same launch also leaving the exact head's ring (fstu_stu_step_lds_pair): ring (B,R,d) in the model dtype receives
 * hist[b,t,:] in slot t % R for the last R positions t <= t_last (R a power of two, 8..1024); slots that a sequence
 * shorter than R does not reach are left as they are (the caller zeroes them).  ring == NULL: as above. */
int fstu_stu_lds_state_ring_from_hist(const void* hist, const float* a, float* state, void* ring, int R, int B, int S,
                                      int d, int t_last, int cap, int dtype, void* stream);

/* ---- STU prefill convolution (approx mode), time-domain form ---------------
 * y[b,t,c] = T(E+O) + T(E-O)  (or T(E+O) if single_branch) with E/O the even-/
 * odd-lag parts of sum_{s<=t} filt[s,c]*xp[b,t-s,c].  xp,y (B,T,d); filt (L,d).
 * Replaces convolve() at flash_stu/utils/stu_utils.py:195-228 + stu.py:120. */
int fstu_stu_conv_direct(const void* xp, const void* filt, void* y, int B, int T, int d, int L,
                         int single_branch, int dtype, void* stream);

/* Exact mode (use_approx=False): the whole filter bank at once.
 *   u_plus[b,t,k,c]  = T( sum_{s<=t} phi[s,k] x[b,t-s,c] )
 *   u_minus[b,t,k,c] = T( sum_{s<=t} (-1)^s phi[s,k] x[b,t-s,c] )   (skipped if NULL)
 * x (B,T,d), phi (L,K), outputs (B,T,K,d).  Replaces convolve(..., use_approx=False)
 * at flash_stu/utils/stu_utils.py:214-228 without expanding x K-fold. */
int fstu_stu_conv_bank(const void* x, const void* phi, void* u_plus, void* u_minus, int B, int T, int d,
                       int L, int K, int dtype, void* stream);

/* ---- STU prefill convolution, FFT form --------------------------------------
 * The reference's own algorithm: rfft of length n, product with the filter's
 * spectrum, irfft, first T outputs kept (flash_stu/utils/stu_utils.py:195-246).
 * Here n is any power of two in 64..16384 with n >= 2T (fstu_fft_length gives the
 * smallest; a circular convolution of that length never wraps into the first T
 * outputs, so the result equals the reference's n = 2^ceil(log2(2L-1))), filters
 * are cut to their first min(L, n/2) taps, and both sign branches come out of one
 * complex inverse transform per channel.
 *
 * fstu_fft_twiddles fills tw (n complex fp32 = 2n floats) with exp(-2 pi i j / n).
 * fstu_stu_fft_filter transforms ncols filter columns (element (s, j) at
 *   filt[s*f_ls + j*f_cs], taps s < taps <= n/2) into spec (ncols, n) complex fp32,
 *   scaled by 1/n, in the transform's internal frequency order; with
 *   single_branch == 0 the spectrum of the (-1)^s branch is folded in as the
 *   imaginary companion.  Approx mode: columns = channels of phi_proj (f_ls = d,
 *   f_cs = 1); exact mode: columns = the K filters of phi (f_ls = K, f_cs = 1).
 *   Replaces the rfft of v at stu_utils.py:213-214 / the cached phi_fft of
 *   flash_stu/modules/stu.py:43-53.
 * fstu_stu_conv_fft: y[b,t,c] = T( T(plus) + T(minus) ) (or T(plus) if
 *   single_branch) for xp, y (B,T,d) and spec (d, n) made with the same n, tw and
 *   single_branch.  Same contract as fstu_stu_conv_direct.
 * fstu_stu_conv_bank_fft: the exact-mode bank, spec (K, n).  x_strides = element
 *   strides {batch, time, channel} of x; u_strides = {batch, time, filter, channel}
 *   of u_plus / u_minus (u_minus may be NULL).  A time stride of 1 (time-major
 *   outputs, the transposed operand of the following contraction) gives fully
 *   coalesced stores.  Same values as fstu_stu_conv_bank. */
int fstu_fft_length(int T);
int fstu_fft_twiddles(float* tw, int n, void* stream);
int fstu_stu_fft_filter(const void* filt, int64_t f_ls, int64_t f_cs, float* spec, const float* tw, int taps,
                        int ncols, int n, int single_branch, int dtype, void* stream);
int fstu_stu_conv_fft(const void* xp, const float* spec, void* y, const float* tw, int B, int T, int d, int n,
                      int single_branch, int dtype, void* stream);
/* The same on strided operands: element (b,t,c) of xp at x_strides[0]*b + x_strides[1]*t + x_strides[2]*c (elements), y
 * likewise.  With a time stride of 1 (time-major slabs (B,d,T)) every load and store of the one-column kernel is
 * coalesced: the form for a few long sequences (transform length 8192 or 16384 and fewer than 512 groups of 8
 * channels x batch rows), where the channel-contiguous kernel leaves compute units idle. */
int fstu_stu_conv_fft_strided(const void* xp, const int64_t* x_strides, const float* spec, void* y, const int64_t* y_strides,
                              const float* tw, int B, int T, int d, int n, int single_branch, int dtype, void* stream);
/* out[b][c][r] = in[b][r][c] for (B,R,C) tensors in either dtype (out must not be in): the copy that hands (B,L,d)
 * activations to fstu_stu_conv_fft_strided as time-major slabs and takes the result back. */
int fstu_transpose(const void* in, void* out, int B, int R, int C, int dtype, void* stream);
int fstu_stu_conv_bank_fft(const void* x, const int64_t* x_strides, const float* spec, void* u_plus, void* u_minus,
                           const int64_t* u_strides, const float* tw, int B, int T, int d, int K, int n, int dtype,
                           void* stream);

/* ---- sliding-window attention ----------------------------------------------
 * KV ring layout: (B,H,cap,hd), absolute position j lives in slot j % cap,
 * cap >= window+1.
 * fstu_kv_append copies k,v of one new token per batch row out of a fused qkv
 * row (B,3*H*hd; q,k,v order) into slot pos % cap.
 * fstu_kv_fill copies the last min(T,cap) positions of a prefill qkv (B,T,3*H*hd)
 * whose first row is absolute position pos0. */
int fstu_kv_append(const void* qkv, void* kring, void* vring, int B, int H, int hd, int cap, int pos,
                   int dtype, void* stream);
int fstu_kv_fill(const void* qkv, void* kring, void* vring, int B, int T, int H, int hd, int cap, int pos0,
                 int dtype, void* stream);

/* One query per (batch,head) at absolute position pos (its own k,v already in
 * the ring) against keys max(0,pos-window)..pos:
 *   s_j = softcap*tanh(q.k_j*hd^-0.5/softcap) - slope[h]*(pos-j)  (softcap<=0: no cap)
 *   out = softmax_j(s) . v   in fp32, rounded to the model dtype.
 * q is read from qkv (B,3*H*hd) columns [0,H*hd); out is (B,H*hd).
 * Replaces flash_attn_func(causal, window_size=(W,0), alibi_slopes, softcap) at
 * flash_stu/modules/attention.py:90-99 for the decode shape. */
int fstu_swa_decode(const void* qkv, const void* kring, const void* vring, void* out, const float* slopes,
                    int B, int H, int hd, int cap, int pos, int window, float softcap, int dtype,
                    void* stream);

/* Same, but first stores the new token's k,v (columns [H*hd,3*H*hd) of the qkv
 * row) into ring slot pos % cap: fstu_kv_append + fstu_swa_decode in one launch. */
int fstu_swa_append_decode(const void* qkv, void* kring, void* vring, void* out, const float* slopes,
                           int B, int H, int hd, int cap, int pos, int window, float softcap, int dtype,
                           void* stream);

/* Prefill form: qkv (B,T,3*H*hd), positions 0..T-1, out (B,T,H*hd). */
int fstu_swa_prefill(const void* qkv, void* out, const float* slopes, int B, int T, int H, int hd,
                     int window, float softcap, int dtype, void* stream);

/* The same prefill attention on the matrix cores (bf16, head dim 64 or 128): S^T = K Q^T and O^T = V^T P^T as
 * v_mfma_f32_16x16x32_bf16 tiles, 16 queries per wave, online softmax in fp32, P carried as a bf16 head plus a bf16
 * remainder so that the second product keeps fp32-P accuracy.  vt_ws is a caller-owned workspace of
 * fstu_swa_prefill_ws_elems(B,T,H,hd) bf16 elements that receives V transposed to (B,H,hd,Tp). */
int64_t fstu_swa_prefill_ws_elems(int B, int T, int H, int hd);
int fstu_swa_prefill_mfma(const void* qkv, void* vt_ws, void* out, const float* slopes, int B, int T, int H, int hd,
                          int window, float softcap, void* stream);

/* ---- sampling --------------------------------------------------------------
 * Per row of logits (B,V): l = clamp(T(logit/temperature), -1e4, 1e4); optional
 * top-k (keep every l >= k-th largest), optional top-p over the survivors
 * (descending order, ties by lower index first; a token is kept iff the
 * probability mass ranked before it is <= top_p), then
 *   do_sample == 0: argmax, lowest index on ties;
 *   do_sample != 0: inverse-CDF draw in index order with the counter-based
 *                   uniform u(seed, step, row).
 * Writes out[b*out_stride] (int64).  top_k <= 0 (or >= V) and top_p outside
 * (0,1) disable the respective filter.  Probabilities are fp32 exponentials
 * relative to the row maximum, summed in float64.
 * Replaces flash_stu/model.py:267-299. */
int fstu_sample(const void* logits, int64_t* out, int64_t out_stride, int B, int V, float temperature,
                int top_k, float top_p, int do_sample, uint64_t seed, int step, int dtype, void* stream);

/* Tied head + greedy pick in one pass: logits[m,:] = T(x[m,:] . W^T) as
 * fstu_linear_decode, and tok_out[m*tok_stride] = argmax_n clamp(T(logit/temperature))
 * with the lowest index on ties (same rule as fstu_sample with do_sample=0).
 * best_ws: rows*64 64-bit words, zero on entry and zero again on return.
 * Replaces lm_head + argmax at flash_stu/model.py:176,268-269,299. */
int fstu_head_argmax(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                     float temperature, void* best_ws, int64_t* tok_out, int64_t tok_stride, int dtype,
                     void* stream);

/* The first half of fstu_head_argmax alone (bf16, K % 256 == 0): the logits, and in best_ws (rows*64 64-bit words, zero on
 * entry) the packed maxima of 64 disjoint subsets of each row: (monotone key of clamp(T(logit/temperature)) << 32) |
 * ~index.  fstu_sample_topk consumes and clears them.  Replaces lm_head at flash_stu/model.py:176. */
int fstu_head_maxima(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                     float temperature, void* best_ws, int dtype, void* stream);

/* The same over a packed copy of the head weight (fstu_pack_rows of the (N,K) embedding; K in {256,512,768,1024,2048},
 * bf16, rows <= 32): one workgroup per CU streams an equal share of the vocabulary against activations it holds in
 * registers, so the activations are not fetched again for every 16 vocabulary rows.  Same logits as fstu_head_maxima up
 * to the summation order over K; the same contract for best_ws.  Replaces lm_head at flash_stu/model.py:176. */
int fstu_head_maxima_packed(const void* x, int ldx, const void* wp, void* logits, int ldy, int rows, int N, int K,
                            float temperature, void* best_ws, void* stream);

/* fstu_sample (do_sample = 1) for bf16 logits and 1 <= top_k <= 64, spread over (V / 2048) x B workgroups instead of one
 * workgroup per row; same draws.  logits: (B, V) rows ldl elements apart; best_ws: the maxima fstu_head_maxima left
 * for these logits at this temperature; samp_ws: fstu_sample_ws_bytes() bytes, zero-initialised once by the caller.
 * best_ws and the counters at the start of samp_ws are zero again when the call completes (the candidate lists behind
 * them keep their last contents, which no later call reads).  1 <= B <= 32, 1024 <= V <= 65536.  The top_k-th largest
 * of a row's 64 maxima bounds the row's top_k-th largest logit from below, so every workgroup keeps only the few
 * tokens above that bound and the last one to finish a row draws from that short list; rows with long plateaus of
 * equal logits are drawn by that workgroup from the whole row instead.  Replaces flash_stu/model.py:267-299. */
int64_t fstu_sample_ws_bytes(void);
int fstu_sample_topk(const void* logits, int64_t ldl, void* best_ws, void* samp_ws, int64_t* out, int64_t out_stride,
                     int B, int V, float temperature, int top_k, float top_p, uint64_t seed, int step, void* stream);

/* fstu_head_argmax for callers that cannot allocate or pass a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * fstu_head_argmax without best_ws: the packed per-row maxima live in a static device array of the library
 * (FSTU_MAX_DECODE_ROWS * 64 64-bit words = 8 KiB, held on every GPU the library runs on until the process ends).
 * rows > FSTU_MAX_DECODE_ROWS is rejected with FSTU_ESHAPE.  The call clears the array with a small fill kernel on
 * `stream` first and allocates nothing (no hipMalloc / hipFree, no allocating library routine).  All calls on one GPU
 * share that GPU's array: calls that overlap on one GPU (different streams or threads) race. */
int fstu_head_argmax_static(const void* x, int ldx, const void* W, void* logits, int ldy, int rows, int N, int K,
                            float temperature, int64_t* tok_out, int64_t tok_stride, int dtype, void* stream);

/* ---- prompt-pass GEMMs on the matrix cores (bf16) ---------------------------
 * C[m,n] = sum_k A[m,k] W[n,k] over M > 16 rows, fp32 accumulation, with the element-wise step that follows the
 * projection in the reference as the epilogue:
 *   mode 0  C = T(acc)                                   c_attn (flash_stu/modules/attention.py:74), x @ M_inputs
 *                                                        (flash_stu/modules/stu.py:87 with W = M_inputs^T)
 *   mode 1  C = T(T(gelu_tanh(T(acc_W))) * T(acc_W2))    gate_proj, up_proj and the gate (flash_stu/modules/swiglu.py:23-26)
 *   mode 2  C = T(R + T(acc))                            c_proj / down_proj and the residual add
 *                                                        (flash_stu/layers/attention_layer.py:57,62)
 * A (M,K) with row stride lda, W and W2 (N,K) contiguous, R / C (M,N) with row strides ldr / ldc (elements).
 * K % 64 == 0, N % 4 == 0, lda % 8 == 0; A, W, W2 16-byte aligned.  C may alias R. */
int fstu_gemm_bf16(const void* A, int64_t lda, const void* W, const void* W2, const void* R, int64_t ldr, void* C,
                   int64_t ldc, int M, int N, int K, int mode, void* stream);
/* The same contraction cut into ksplit slices of K, for a long K with few output tiles (down_proj of a decode step over
 * 17..32 rows, flash_stu/modules/swiglu.py:28): partial (ksplit,M,N) fp32 receives the unrounded slice sums, which
 * fstu_add_rmsnorm (delta_mode 1, nslices = ksplit) adds into the residual stream as T(x + T(sum)).
 * K % (64*ksplit) == 0, ksplit 1..64. */
int fstu_gemm_bf16_splitk(const void* A, int64_t lda, const void* W, float* partial, int M, int N, int K, int ksplit,
                          void* stream);

/* General contraction for what fstu_gemm_bf16 does not take: fp32 (the reference's fp32 configuration,
 * flash_stu/model.py:108-205 with torch_dtype float32: every nn.Linear of the prompt pass), bf16 shapes with
 * K % 32 != 0 or unaligned rows, and operands given by strides (phi @ M_filters, flash_stu/modules/stu.py:88; the
 * fp32 slabs of exact mode, stu.py:107-120).  C (M,N; row stride ldc) = T(A W^T), A element (m,k) at A[m*sam + k*sak],
 * W element (n,k) at W[n*swn + k*swk] (strides in elements, positive); fp32 accumulation on the fp32 matrix
 * instruction, one rounding to `dtype`.  Any M, N, K >= 1. */
int fstu_gemm_any(const void* A, int64_t sam, int64_t sak, const void* W, int64_t swn, int64_t swk, void* C, int64_t ldc,
                  int M, int N, int K, int dtype, void* stream);

/* The contraction of the exact-mode STU operator (flash_stu/modules/stu.py:107-120: tensordot of U+- (B,L,K,d) with
 * M_phi+- (K,d,d) over (K,d)) with U stored as the filter-bank kernel writes it, time-major: nbatch slabs A[b] of shape
 * (K, M) — the reduction index slowest, M contiguous, row stride lda, slab stride batch_stride_a (elements) — against
 * W (N, K) row-major (M_phi flattened to (K*d, N) and transposed once at model-prepare time):
 *   mode 0  C[b] = T(A[b]^T W^T)            mode 2  C[b] = T(R[b] + T(A[b]^T W^T))   (the sum of the two sign branches)
 * C, R (nbatch, M, N) with row strides ldc / ldr and slab strides batch_stride_c / batch_stride_r; C may alias R.
 * M % 128 == 0, K % 64 == 0, N % 4 == 0, lda % 8 == 0, K*lda*2 and N*K*2 below 4 GB; A, W 16-byte aligned. */
int fstu_gemm_bf16_ta(const void* A, int64_t lda, int64_t batch_stride_a, const void* W, const void* R, int64_t ldr,
                      int64_t batch_stride_r, void* C, int64_t ldc, int64_t batch_stride_c, int M, int N, int K, int nbatch,
                      int mode, void* stream);

/* ---- dense LDS (mini_stu/lds.py:95-101) ------------------------------------
 * T_steps consecutive steps with the fp32 state h (Bt,S) carried in place:
 *   h <- h*A + x_t @ Bm ;  y_t = T(h @ Cm)
 * x (T_steps,Bt,d_in), y (T_steps,Bt,d_out) in the model dtype; A (S) fp32;
 * Bm (d_in,S), Cm (S,d_out) in the model dtype.  S <= 256. */
int fstu_lds_steps(float* h, const void* x, const float* A, const void* Bm, const void* Cm, void* y,
                   int T_steps, int Bt, int d_in, int S, int d_out, int dtype, void* stream);

/* The same loop over a whole sequence on the matrix cores (bf16): blocks of 128 positions run in parallel (x_t @ Bm
 * does not depend on the state), a short chain hands the state from block to block.  Weights are given TRANSPOSED:
 * BmT (S,d_in), CmT (d_out,S).  ws: fstu_lds_sequence_ws_floats(T,Bt,S) floats, owned by the caller (any contents; calls
 * that share a workspace must not overlap).  d_in % 32 == 0,
 * S % 32 == 0, S <= 256, d_out % 16 == 0.  Same values as fstu_lds_steps up to the fp32 summation order; a sequence
 * split at a multiple of 128 positions into two calls gives bit-identical outputs and states.  x is read once: a
 * block takes the state that enters it from what the blocks in front of it publish inside the same launch; that wait
 * is bounded, and fstu_lds_sequence_status (a synchronous read) returns *err_out = 1 when it ran out in the last call
 * on that workspace (the outputs of that call are then not valid), 0 otherwise. */
size_t fstu_lds_sequence_ws_floats(int T, int Bt, int S);
int fstu_lds_sequence_status(const float* ws, int* err_out);
int fstu_lds_sequence(float* h, const void* x, const float* A, const void* BmT, const void* CmT, void* y, float* ws,
                      int T, int Bt, int d_in, int S, int d_out, void* stream);

/* ---- packed weights -------------------------------------------------------------
 * Packed layout of an (N,K) bf16 row-major weight, K % 32 == 0 (fstu_pack_rows):
 *   Wp[tile][kstep][lane][8],  tile = n/16, kstep = k/32, lane = 16*g + r,
 *   element e of lane (r,g) = W[16*tile + r][32*kstep + 8*g + e]; rows >= N are zero
 * i.e. the A-operand fragment of v_mfma_f32_16x16x32_bf16: one wave load reads 1 KB of contiguous memory.
 * fstu_packed_elems(N,K) is the number of bf16 elements of the packed copy. */
int64_t fstu_packed_elems(int N, int K);
int fstu_pack_rows(const void* W, void* Wp, int N, int K, void* stream);

/* Gate/up projection with the GLU epilogue over packed weights, one workgroup per CU with equal bytes each
 * (4-feature granularity) and every weight fragment in flight from the first instruction:
 *   act[r,f] = T( T(gelu_tanh(T(h[r,:].Wg[f,:]))) * T(h[r,:].Wu[f,:]) ),  rows <= 16 (32: below), bf16.
 * Same contract as fstu_glu_decode (flash_stu/modules/swiglu.py:23-26); wp_* from fstu_pack_rows.
 * fstu_glu_packed_supported tells whether a shape is covered (d in {256,512,768,1024,2048}, I % 4 == 0).
 * 17..32 rows (fstu_mlp_packed_rows32_supported: such a d, I % 512 == 0): fstu_glu_packed and fstu_down_packed_splitk
 * take them as two row tiles per weight fragment, so every weight is still read once; of the launches with a norm
 * prologue fstu_glu_packed_norm and fstu_linear_packed take them too (see there), fstu_linear_packed_res stays at 16 rows. */
int fstu_glu_packed_supported(int rows, int d, int I);
int fstu_mlp_packed_rows32_supported(int rows, int d, int I);
int fstu_glu_packed(const void* h, int ldh, const void* wp_gate, const void* wp_up, void* act, int ldact, int rows,
                    int I, int d, void* stream);
/* The same launch with the sub-layer's residual add and mlp_norm as its prologue (stu_layer.py:93-96,
 * attention_layer.py:59-62): x' = T(x_in + delta) (delta may be NULL), h = rmsnorm(x') * norm_w recomputed by every
 * workgroup while its weight loads are in flight; x' is stored to x_out (may be NULL; must not alias x_in).
 * 17..32 rows: x_in is the stream with the sub-layer's output already added (fstu_linear_packed_add,
 * fstu_stu_step_lds_pair_add), delta and x_out must be NULL; the norm is formed in the matrix-core fragments. */
int fstu_glu_packed_norm(const void* x_in, const void* delta, void* x_out, const void* norm_w, float eps,
                         const void* wp_gate, const void* wp_up, void* act, int ldact, int rows, int I, int d,
                         void* stream);

/* y = T(x W^T) over packed W (N,K) with the same balanced launch; with norm_w != NULL, x is the residual stream
 * (dense rows) and h = rmsnorm(x) * norm_w is formed in the prologue (the sub-layer norm of stu_layer.py:81 /
 * attention_layer.py:53 fused into c_attn / M_inputs).  K in {256,512,768,1024,2048}, N % 4 == 0, bf16, rows <= 32
 * (17..32: the second 16 as another row tile of the same weight fragments, and the norm formed in those fragments
 * instead of in LDS). */
int fstu_linear_packed(const void* x, int ldx, const void* norm_w, float eps, const void* wp, void* y, int ldy,
                       int rows, int N, int K, void* stream);
/* The same projection joining the residual stream (flash_stu/layers/attention_layer.py:57, x = x + attn(attn_norm(x))
 * with c_proj as the projection): res_out = T(res_in + T(x W^T)), rows of stride N in both; res_out may be res_in.
 * rows <= 32, N % 8 == 0, K as above, bf16. */
int fstu_linear_packed_add(const void* x, int ldx, const void* wp, const void* res_in, void* res_out, int rows, int N,
                           int K, void* stream);
/* Split-K form of the down projection over packed weights (reference: flash_stu/modules/swiglu.py:22-29, down_proj):
 * partial receives *ksplit_io fp32 slices (slice, rows, d) that fstu_add_rmsnorm(delta_mode 1) or the norm prologue of
 * the next projection sums in slice order.  *ksplit_io on entry: slices wanted (4, 8 or 16; anything else: 16); on
 * return: slices written.  d % 16 == 0, I % (32 * slices) == 0, rows <= 32, bf16.  Same values as
 * fstu_linear_decode_splitk up to the summation order. */
int fstu_down_packed_splitk(const void* act, int ldact, const void* wp_down, float* partial, int rows, int d, int I,
                            int* ksplit_io, void* stream);

/* y = T(h W^T) over packed W (N,K) with h = rmsnorm(x') * norm_w, x' = T(x_in + T(sum of nslices <= 4 fp32 slices)):
 * the residual add + RMSNorm between the MLP of one layer and the first projection of the next
 * (flash_stu/layers/stu_layer.py:93-97 followed by attention_layer.py:53-57), folded into that projection.  x' goes to
 * x_out (must not alias x_in).  K % 256 == 0, rows*K/8 <= 1024, rows <= 16, bf16. */
int fstu_linear_packed_res(const void* x_in, const float* partial, int nslices, void* x_out, const void* norm_w, float eps,
                           const void* wp, void* y, int ldy, int rows, int N, int K, void* stream);

/* ---- whole decode step -----------------------------------------------------
 * One call launches every kernel of one token step for all layers: embedding of
 * the input token, the layer stack against its decode state, final norm, tied
 * head, and sampling of the next token.  It is the body of the loop at
 * flash_stu/model.py:245-302 for steps after the first, with the per-layer state
 * the reference lacks for STU layers (flash_stu/layers/stu_layer.py:99-120).
 * The descriptors only carry device pointers owned by the caller. */
typedef struct {
  int kind;                 /* 0: STU layer (approx mode), 1: attention layer */
  const void* norm1_w;      /* stu_norm / attn_norm weight (d) */
  const void* mlp_norm_w;   /* (d) */
  const void* w_gate;       /* (I,d) */
  const void* w_up;         /* (I,d) */
  const void* w_down;       /* (d,I) */
  /* STU */
  const void* m_inputs_t;   /* (d,d): M_inputs transposed, [out][in] */
  const void* filt;         /* (L,d) phi_proj, model dtype       (history mode) */
  void* hist;               /* (B,hist_cap,d) x_proj history      (history mode) */
  const float* lds_a;       /* (S)                                (lds mode) */
  const float* lds_ce;      /* (S,d) even-lag output weights      (lds mode) */
  const float* lds_co;      /* (S,d) odd-lag output weights on the other bank, or NULL: y = T(2E) (lds mode) */
  float* lds_state;         /* (B,2,S,d)                          (lds mode) */
  void* lds_ring;           /* (B,lds_fir_taps,d) last projected inputs, model dtype, or NULL (lds mode, with lds_co) */
  const float* lds_fir;     /* (lds_fir_taps,d) phi_proj minus the fitted filter on the first lags, or NULL */
  float* lds_ocache;        /* (B,d) fp32 or NULL: the odd-lag sum handed from step to step (fstu_stu_step_lds_pair_cached),
                               primed for the first decode position by fstu_stu_step_lds_prime; used by the 17..32-row step */
  /* attention */
  const void* w_qkv;        /* (3d,d) */
  const void* w_proj;       /* (d,d) */
  void* kring;              /* (B,H,kv_cap,hd) */
  void* vring;
  const float* slopes;      /* (H) */
  /* packed copies (fstu_pack_rows) for the fused bf16 step; all NULL = not available */
  const void* wp_gate;
  const void* wp_up;
  const void* wp_down;
  const void* wp_m_inputs;  /* packed M_inputs^T */
  const void* wp_qkv;
  const void* wp_proj;
} fstu_layer_desc;

typedef struct {
  int dtype;
  int B, d, I, V, n_layers, n_heads, head_dim;
  int window, kv_cap;
  int L, hist_cap;
  int stu_mode;             /* 0: history, 1: lds */
  int lds_S;
  int lds_fir_taps;         /* taps of the layers' lds_fir (a power of two, 8..1024), 0: none */
  int single_branch;        /* use_hankel_L */
  int ksplit_down;          /* K split of the down projection (partial holds ksplit_down*B*d floats) */
  int hist_nsplit_max;      /* eo holds hist_nsplit_max*2*B*d floats */
  int row0;                 /* index of this descriptor's first row in the caller's batch (keys the sampling stream) */
  float eps, softcap;
  const void* emb;          /* (V,d) tied embedding / head */
  const void* final_norm_w; /* (d) */
  const fstu_layer_desc* layers;   /* host array of n_layers entries */
  /* workspaces, model dtype unless noted */
  void* x;                  /* (B,d) residual stream */
  void* h;                  /* (B,d) normalised activations */
  void* qkv;                /* (B,3d) */
  void* attn;               /* (B,d) */
  void* act;                /* (B,I) */
  void* xp;                 /* (B,d) */
  void* y;                  /* (B,d) */
  float* partial;           /* fp32 */
  float* eo;                /* fp32 */
  void* logits;             /* (B,V) */
  void* best;               /* max(B,16)*64 64-bit words, zero-initialised once by the caller */
  void* samp_ws;            /* fstu_sample_ws_bytes() bytes, zero-initialised once by the caller, or NULL: top-k sampling
                               then runs one workgroup per row (fstu_sample) instead of fstu_sample_topk */
  const void* wp_emb;       /* packed tied head (fstu_pack_rows of emb) or NULL: the head then reads emb row-major */
  void* x2;                 /* (B,d) second residual buffer (the stream ping-pongs x <-> x2); NULL: the add + norm
                               between sub-layers runs as launches of its own */
  int glu_packed;           /* != 0: layers with wp_gate and wp_up run their gate/up projection through fstu_glu_packed */
  int down_packed;          /* != 0: layers with wp_down use fstu_down_packed_splitk (16 slices: partial must hold
                               max(ksplit_down,16)*B*d floats) */
  int merge_norm;           /* != 0 (needs glu_packed, down_packed, x2, lds mode, wp_gate/up/down everywhere and wp_qkv on
                               attention layers, B*d <= 8192): the down projection leaves 4 split-K slices and the next
                               layer's first projection adds and normalises them in its prologue
                               (fstu_stu_res_inproj_step / fstu_linear_packed_res); one add+norm launch less per layer */
} fstu_model_desc;

/* tok_in[b*tok_stride] is the token at absolute position pos; the sampled next
 * token is written to tok_out[b*tok_stride].  `step` indexes the sampling
 * stream.  Sampling arguments as in fstu_sample. */
int fstu_decode_step(const fstu_model_desc* m, const int64_t* tok_in, int64_t* tok_out, int64_t tok_stride,
                     int pos, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                     int step, void* stream);

/* One decode step captured as a HIP graph that can be replayed for every position:
 * the position-dependent kernels read {position, sampling step} from `dyn`, a
 * device int[2] the caller sets before the first launch; every launch feeds
 * tokens[:, dyn[0]], writes tokens[:, dyn[0]+1] and then advances both counters.
 * Requires the recurrence (lds) STU state.  `stream` must be a non-default stream;
 * capture happens on it inside fstu_decode_graph_create (no memset nodes are
 * recorded).  pos0 is the value the caller stores in dyn[0] before the first launch: with the recurrence STU state
 * two graphs are captured, one per parity of the position (their STU launches carry the parity as an argument
 * instead of reading dyn first), and launch n replays the one for pos0 + n; a caller that rewrites dyn[0] creates a
 * new graph.  nsteps (1..64) consecutive decode steps are captured into one graph, so that one launch produces
 * nsteps tokens per sequence (the cost of starting a graph is paid once per nsteps tokens).  No counterpart in the
 * reference. */
int fstu_decode_graph_create(const fstu_model_desc* m, int64_t* tokens, int64_t tok_stride, int* dyn, int pos0,
                             int nsteps, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                             void* stream, void** graph_out);
int fstu_decode_graph_launch(void* graph, void* stream);
/* Tells the graph which position its next launch will process: needed when other graphs (of another length) over the
 * same tokens and `dyn` have advanced the device-side position since this graph's last launch.  A graph of an even
 * number of steps is captured for one parity of its first position only; seeking it to the other parity is rejected. */
int fstu_decode_graph_seek(void* graph, long long next_pos);
int fstu_decode_graph_destroy(void* graph);

/* ---- live kernel timing (measurement aid; no counterpart in the reference) ----
 * Between fstu_prof_begin and fstu_prof_end every launch of one kernel class
 * inside fstu_decode_step is bracketed by HIP events on the launch stream
 * (at most max_launches of them; events are created and destroyed by these two
 * calls).  fstu_prof_end waits for the events and returns the summed kernel
 * time and the number of launches.  Classes: 1 gate/up GLU, 2 down projection,
 * 3 head, 4 attention (append+decode), 5 STU step, 6 d-by-d projections and
 * QKV, 7 embed/add/RMSNorm, 8 sampling.  Not thread-safe. */
int fstu_prof_begin(int kernel_class, int max_launches);
int fstu_prof_end(double* total_ms, int* launches);
/* The gate/up GLU projection (fstu_glu_decode) of every layer of `m`, `reps` times back to back on `stream`
 * between two HIP events; returns the elapsed time and launch count.  Synchronises on the second event. */
/* Plain copy kernel of a known size: the reference launch against which FETCH_SIZE / WRITE_SIZE counter readings
 * of the other kernels are scaled. */
int fstu_prof_copy(void* dst, const void* src, size_t bytes, void* stream);
int fstu_prof_glu_loop(const fstu_model_desc* m, int reps, double* total_ms, int* launches, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHSTU_HIP_H */
