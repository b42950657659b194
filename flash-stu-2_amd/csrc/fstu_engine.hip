// Host-side driver of one decode step: the launch sequence over the layer
// stack, with every residual add fused into the RMSNorm that follows it.
#include "fstu_common.h"

#define STEP(call)          \
  do {                      \
    int rc__ = (call);      \
    if (rc__ != 0) return rc__; \
  } while (0)

// ---------------------------------------------------------------- live kernel timing
// Optional: HIP events recorded around every launch of one kernel class inside
// fstu_decode_step, on the stream the kernels run on.
enum { PC_NONE = 0, PC_GLU = 1, PC_DOWN = 2, PC_HEAD = 3, PC_SWA = 4, PC_STU = 5, PC_PROJ = 6, PC_NORM = 7, PC_SAMPLE = 8, PC_NCLASS = 9 };
static int g_prof_class = PC_NONE;
static hipEvent_t* g_prof_ev = nullptr;
static int g_prof_cap = 0, g_prof_n = 0;

extern "C" int fstu_prof_begin(int kernel_class, int max_launches) {
  FSTU_REQUIRE(kernel_class > PC_NONE && kernel_class < PC_NCLASS && max_launches > 0, FSTU_EARG, "fstu_prof_begin: bad class %d / capacity %d", kernel_class, max_launches);
  FSTU_REQUIRE(g_prof_ev == nullptr, FSTU_EARG, "fstu_prof_begin: already profiling");
  g_prof_ev = new hipEvent_t[2 * (size_t)max_launches];
  for (int i = 0; i < 2 * max_launches; ++i) {
    hipError_t e = hipEventCreate(&g_prof_ev[i]);
    if (e != hipSuccess) { fstu_set_error("fstu_prof_begin: hipEventCreate: %s", hipGetErrorString(e)); return (int)e; }
  }
  g_prof_class = kernel_class;
  g_prof_cap = max_launches;
  g_prof_n = 0;
  return FSTU_OK;
}

extern "C" int fstu_prof_end(double* total_ms, int* launches) {
  FSTU_REQUIRE(g_prof_ev != nullptr && total_ms && launches, FSTU_EARG, "fstu_prof_end: not profiling");
  double tot = 0.0;
  for (int i = 0; i < g_prof_n; ++i) {
    (void)hipEventSynchronize(g_prof_ev[2 * i + 1]);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, g_prof_ev[2 * i], g_prof_ev[2 * i + 1]);
    tot += ms;
  }
  for (int i = 0; i < 2 * g_prof_cap; ++i) (void)hipEventDestroy(g_prof_ev[i]);
  delete[] g_prof_ev;
  g_prof_ev = nullptr;
  *total_ms = tot;
  *launches = g_prof_n;
  g_prof_class = PC_NONE;
  g_prof_cap = g_prof_n = 0;
  return FSTU_OK;
}

// The gate/up GLU projection of every layer, `reps` times back to back on `stream`, between two HIP events:
// average duration of the dominant decode kernel at its real shapes and weights.
extern "C" int fstu_prof_glu_loop(const fstu_model_desc* m, int reps, double* total_ms, int* launches, void* stream) {
  FSTU_REQUIRE(m && total_ms && launches && reps >= 1, FSTU_EARG, "fstu_prof_glu_loop: bad arguments");
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { fstu_set_error("fstu_prof_glu_loop: hipEventCreate failed"); return FSTU_EARG; }
  int rc = 0, n = 0;
  // the same kernel the step launches for this projection
  auto glu = [&](int l) {
    const fstu_layer_desc& L = m->layers[l];
    if (m->dtype == FSTU_BF16 && m->glu_packed && L.wp_gate && L.wp_up && fstu_glu_packed_supported(m->B, m->d, m->I)) {
      if (m->x2)   // as in the step: residual add + mlp_norm as the prologue
        return fstu_glu_packed_norm(m->x, m->y, m->x2, L.mlp_norm_w, m->eps, L.wp_gate, L.wp_up, m->act, m->I, m->B, m->I, m->d, stream);
      return fstu_glu_packed(m->h, m->d, L.wp_gate, L.wp_up, m->act, m->I, m->B, m->I, m->d, stream);
    }
    return fstu_glu_decode(m->h, m->d, L.w_gate, L.w_up, m->act, m->I, m->B, m->I, m->d, m->dtype, stream);
  };
  for (int l = 0; l < m->n_layers && rc == 0; ++l) rc = glu(l);   // warm-up pass
  (void)hipEventRecord(e0, (hipStream_t)stream);
  for (int r = 0; r < reps && rc == 0; ++r)
    for (int l = 0; l < m->n_layers && rc == 0; ++l, ++n) rc = glu(l);
  (void)hipEventRecord(e1, (hipStream_t)stream);
  (void)hipEventSynchronize(e1);
  float ms = 0.f;
  (void)hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *total_ms = ms;
  *launches = n;
  return rc;
}

// A plain copy of `bytes` bytes (16-byte granules): the calibration launch for hardware traffic counters, whose
// FETCH_SIZE / WRITE_SIZE readings for this kernel are known in advance.
__global__ void __launch_bounds__(256) prof_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

extern "C" int fstu_prof_copy(void* dst, const void* src, size_t bytes, void* stream) {
  FSTU_REQUIRE(dst && src && bytes % 16 == 0 && fstu_aligned(dst, 16) && fstu_aligned(src, 16), FSTU_EARG,
               "fstu_prof_copy: pointers and size must be 16-byte multiples");
  hipLaunchKernelGGL(prof_copy_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, (uint4*)dst, (const uint4*)src, bytes / 16);
  FSTU_CHECK_LAUNCH("fstu_prof_copy");
  return FSTU_OK;
}

#define TIMED(cls, call)                                                                        \
  do {                                                                                          \
    const bool t__ = (g_prof_class == (cls)) && g_prof_n < g_prof_cap;                          \
    if (t__) (void)hipEventRecord(g_prof_ev[2 * g_prof_n], (hipStream_t)stream);                    \
    int rc__ = (call);                                                                          \
    if (t__) { (void)hipEventRecord(g_prof_ev[2 * g_prof_n + 1], (hipStream_t)stream); ++g_prof_n; }  \
    if (rc__ != 0) return rc__;                                                                 \
  } while (0)

// recurrence step on m->xp: both sign branches rounded separately when the layer carries odd-lag weights
// (stream_x: the residual stream; the step then adds its output to it in place instead of leaving it in m->y)
// (wide: the 17..32-row step, which hands the odd-lag sum from step to step where the layer carries lds_ocache)
static int stu_step(const fstu_layer_desc& L, const fstu_model_desc* m, int pos, const int* dyn, const int* pos_dyn, void* stream,
                    void* stream_x = nullptr, bool wide = false) {
  if (L.lds_co)
    return fstu_stu_step_lds_pair_dyn(L.lds_state, m->xp, m->d, L.lds_a, L.lds_ce, L.lds_co, L.lds_ring, L.lds_fir,
                                      L.lds_fir ? m->lds_fir_taps : 0, stream_x ? stream_x : m->y, m->d, m->B, m->lds_S, m->d, pos,
                                      dyn, pos_dyn, m->dtype, stream, stream_x, wide ? L.lds_ocache : nullptr);
  if (stream_x) return FSTU_EARG;
  return fstu_stu_step_lds_dyn(L.lds_state, m->xp, m->d, L.lds_a, L.lds_ce, m->y, m->d, m->B, m->lds_S, m->d, pos, dyn, m->dtype,
                               stream);
}

static int hist_nsplit(int nlags, int maxsplit) {
  int n = nlags / 64;
  if (n < 1) n = 1;
  if (n > 16) n = 16;
  if (n > maxsplit) n = maxsplit;
  return n;
}

// While a graph is captured for one parity of the position, the STU launches get that parity as a plain argument
// instead of reading the device-side position first: their state addresses then depend on nothing, which takes one
// dependent trip to memory (about 1 us) off each of them.  -1: no override.
static thread_local int g_stu_parity = -1;
static inline const int* stu_dyn(const int* dyn) { return g_stu_parity >= 0 ? nullptr : dyn; }
static inline int stu_pos(int pos) { return g_stu_parity >= 0 ? g_stu_parity : pos; }

// Inside a graph of several greedy steps the reduction of one step's packed maxima (token store, position advance) and
// the next step's embedding + norm are one launch.  g_chain_prev: this step starts with that launch; g_chain_next:
// this step's head leaves its maxima for the next step.
static thread_local bool g_chain_prev = false, g_chain_next = false;
static bool chain_ok(const fstu_model_desc* m, int do_sample, const int* dyn) {
  return dyn && !do_sample && m->best && m->dtype == FSTU_BF16 && fstu_head_argmax_fused_pick(m->h, m->d, m->emb, m->d, m->dtype) &&
         fstu_finish_embed_supported(m->B, m->d, m->emb, m->x, m->layers[0].norm1_w, m->h);
}

// top-k sampling spread over the chip: needs the head kernel that leaves the packed maxima and the sampler's workspace
static bool sample_spread_ok(const fstu_model_desc* m, int do_sample, int top_k) {
  return do_sample && m->best && m->samp_ws && fstu_sample_topk_ok(m->B, m->V, top_k, m->dtype) &&
         fstu_head_argmax_fused_pick(m->h, m->d, m->emb, m->d, m->dtype);
}

// 17..32 rows: the MLP, where nearly all the weight bytes are, runs once over all rows on the tiled matrix-core kernel
// (gate/up with the GLU epilogue, split-K down projection), so every MLP weight is read once per step; the
// STU recurrence and the window attention, per-row operators, run over all rows in one launch each, and the small
// projections and the head keep their 16-row kernels and run on the two halves of the rows in turn.  bf16 and the recurrence (lds) STU state only.
static int decode_step_wide(const fstu_model_desc* m, const int64_t* tok_in, int64_t* tok_out, int64_t tok_stride, int pos,
                            float temperature, int top_k, float top_p, int do_sample, uint64_t seed, int step, int* dyn,
                            void* stream) {
  const int B = m->B, d = m->d, I = m->I, dt = m->dtype, R = FSTU_MAX_DECODE_ROWS;
  FSTU_REQUIRE(dt == FSTU_BF16 && m->stu_mode == 1 && d % 256 == 0 && I % 64 == 0, FSTU_ESHAPE,
               "fstu_decode_step: more than %d rows need bf16, the recurrence STU state, d %% 256 == 0 and I %% 64 == 0", R);
  FSTU_REQUIRE(m->qkv && m->attn && m->y && m->xp && m->partial, FSTU_ENULL, "fstu_decode_step: incomplete model descriptor");
  // K slices of the down projection: its d/128 output tiles times the slices should cover the chip; the partial-sum
  // buffer holds at least 16 slices
  int ks = 16;
  while (ks > 1 && (I % (64 * ks) != 0 || (d / 128) * ks > 512)) ks >>= 1;
  const bool packed_mlp = fstu_mlp_packed_rows32_supported(B, d, I) && I / 512 <= 96;
  const size_t esz = 2;
  auto rows_of = [&](int c) { return c == 0 ? R : B - R; };
  auto at = [&](void* p, int c, size_t per_row) { return (void*)((char*)p + (size_t)c * R * per_row * esz); };
  // y = x W^T over all rows: one launch with two row tiles per weight fragment where the operands allow it, else the
  // 16-row kernel on the two halves of the rows in turn
  auto proj = [&](void* x, int ldx, const void* W, void* y, int ldy, int N, int K) -> int {
    if (fstu_linear_rows32_ok(x, ldx, W, K, dt)) return fstu_linear_rows32(x, ldx, W, y, ldy, B, N, K, 1.0f, nullptr, stream);
    for (int c = 0; c < 2; ++c) {
      int rc = fstu_linear_decode(at(x, c, ldx), ldx, W, at(y, c, ldy), ldy, rows_of(c), N, K, dt, stream);
      if (rc) return rc;
    }
    return FSTU_OK;
  };
  TIMED(PC_NORM, fstu_embed_rmsnorm(tok_in, tok_stride, m->emb, m->x, m->layers[0].norm1_w, m->h, B, d, m->V, m->eps, dt, stream, dyn));
  // raw: the residual stream in m->x has the previous layer's MLP output added but is not normalised yet (m->h is
  // stale); the layer's first projection, over packed weights, then forms its norm in its own fragments
  bool raw = false;
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    const void* xin = raw ? m->x : m->h;
    const void* nw1 = raw ? L.norm1_w : nullptr;
    // Where the layer's MLP streams packed weights, the sub-layer's last launch adds its output to the residual stream
    // itself (m->x in place) and the gate/up launch normalises the stream in its own fragments: no add+norm launch
    // between them.
    const bool join = packed_mlp && L.wp_gate && L.wp_up && (L.kind == 0 ? L.lds_co != nullptr : L.wp_proj != nullptr);
    if (L.kind == 0) {
      // in-projection on the two halves of the rows (16-row kernel), then one recurrence launch over all rows
      if (packed_mlp && L.wp_m_inputs) TIMED(PC_PROJ, fstu_linear_packed(xin, d, nw1, m->eps, L.wp_m_inputs, m->xp, d, B, d, d, stream));
      else TIMED(PC_PROJ, proj(m->h, d, L.m_inputs_t, m->xp, d, d, d));
      TIMED(PC_STU, stu_step(L, m, stu_pos(pos), stu_dyn(dyn), dyn, stream, join ? m->x : nullptr, true));
    } else {
      if (packed_mlp && L.wp_qkv) TIMED(PC_PROJ, fstu_linear_packed(xin, d, nw1, m->eps, L.wp_qkv, m->qkv, 3 * d, B, 3 * d, d, stream));
      else TIMED(PC_PROJ, proj(m->h, d, L.w_qkv, m->qkv, 3 * d, 3 * d, d));
      TIMED(PC_SWA, fstu_swa_decode_impl(m->qkv, L.kring, L.vring, m->attn, L.slopes, B, m->n_heads, m->head_dim, m->kv_cap, pos,
                                         m->window, m->softcap, 1, dyn, dt, stream));
      if (join) TIMED(PC_PROJ, fstu_linear_packed_add(m->attn, d, L.wp_proj, m->x, m->x, B, d, d, stream));
      else if (packed_mlp && L.wp_proj) TIMED(PC_PROJ, fstu_linear_packed(m->attn, d, nullptr, 0.f, L.wp_proj, m->y, d, B, d, d, stream));
      else TIMED(PC_PROJ, proj(m->attn, d, L.w_proj, m->y, d, d, d));
    }
    const void* next_w = (l + 1 < m->n_layers) ? m->layers[l + 1].norm1_w : m->final_norm_w;
    // the MLP over packed weights where the model holds them (contiguous streams, one workgroup per compute unit with
    // equal bytes each: measured 33 against 46 us for the 201 MB of a 2048-d gate/up pair), else the tiled GEMM
    int nsl = ks;
    if (join) {
      TIMED(PC_GLU, fstu_glu_packed_norm(m->x, nullptr, nullptr, L.mlp_norm_w, m->eps, L.wp_gate, L.wp_up, m->act, I, B, I, d, stream));
    } else {
      TIMED(PC_NORM, fstu_add_rmsnorm(m->x, m->y, 0, 1, 0, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
      if (packed_mlp && L.wp_gate && L.wp_up) TIMED(PC_GLU, fstu_glu_packed(m->h, d, L.wp_gate, L.wp_up, m->act, I, B, I, d, stream));
      else TIMED(PC_GLU, fstu_gemm_bf16(m->h, d, L.w_gate, L.w_up, nullptr, 0, m->act, I, B, I, d, 1, stream));
    }
    if (packed_mlp && L.wp_down) {
      nsl = 16;
      TIMED(PC_DOWN, fstu_down_packed_splitk(m->act, I, L.wp_down, m->partial, B, d, I, &nsl, stream));
    } else {
      TIMED(PC_DOWN, fstu_gemm_bf16_splitk(m->act, I, L.w_down, m->partial, B, d, I, ks, stream));
    }
    // The split-K slices join the stream in a launch that the whole chip shares (one workgroup per row would fetch
    // 131 KB each); where the next layer's first projection streams packed weights it forms the norm itself
    raw = false;
    if (packed_mlp && l + 1 < m->n_layers && d % 4 == 0) {
      const fstu_layer_desc& Nx = m->layers[l + 1];
      raw = Nx.kind == 0 ? Nx.wp_m_inputs != nullptr : Nx.wp_qkv != nullptr;
    }
    if (raw) TIMED(PC_NORM, fstu_add_slices(m->x, m->partial, nsl, B, d, dt, stream));
    else TIMED(PC_NORM, fstu_add_rmsnorm(m->x, m->partial, 1, nsl, 0, next_w, m->h, B, d, m->eps, dt, stream));
  }
  if (sample_spread_ok(m, do_sample, top_k)) {
    // the head leaves each row's packed maxima, the sampler spreads every row over the chip and advances {pos, step}
    // over the packed copy of the embedding where the model holds one: a workgroup keeps the activations in registers
    // instead of fetching the 32 rows again for every 16 vocabulary rows (40 against 75 us at 2048-d)
    if (m->wp_emb && fstu_glu_packed_supported(R, d, m->V))
      TIMED(PC_HEAD, fstu_head_maxima_packed(m->h, d, m->wp_emb, m->logits, m->V, B, m->V, d, temperature, m->best, stream));
    else if (fstu_linear_rows32_ok(m->h, d, m->emb, d, dt))
      TIMED(PC_HEAD, fstu_linear_rows32(m->h, d, m->emb, m->logits, m->V, B, m->V, d, temperature, m->best, stream));
    else
      for (int c = 0; c < 2; ++c)
        TIMED(PC_HEAD, fstu_head_maxima(at(m->h, c, d), d, m->emb, at(m->logits, c, (size_t)m->V), m->V, rows_of(c), m->V, d, temperature,
                                        (char*)m->best + (size_t)c * R * 64 * 8, dt, stream));
    TIMED(PC_SAMPLE, fstu_sample_topk_dyn(m->logits, m->V, m->best, m->samp_ws, tok_out, tok_stride, B, m->V, temperature, top_k, top_p,
                                          seed, step, m->row0, dyn, 1, stream));
    return FSTU_OK;
  }
  TIMED(PC_HEAD, proj(m->h, d, m->emb, m->logits, m->V, m->V, d));
  TIMED(PC_SAMPLE, fstu_sample_dyn(m->logits, tok_out, tok_stride, B, m->V, temperature, top_k, top_p, do_sample, seed, step, m->row0,
                                   dyn, dt, stream));
  if (dyn) STEP(fstu_advance_dyn(dyn, stream));
  return FSTU_OK;
}

// dyn == nullptr: pos/step come from the host arguments.  dyn != nullptr (graph capture): every position-dependent
// kernel reads {pos, step} from that device int[2]; tok_in/tok_out are then the bases of token columns 0 and 1.
static int decode_step_impl(const fstu_model_desc* m, const int64_t* tok_in, int64_t* tok_out, int64_t tok_stride,
                            int pos, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                            int step, int* dyn, void* stream) {
  FSTU_REQUIRE(m && tok_in && tok_out, FSTU_ENULL, "fstu_decode_step: null pointer");
  FSTU_REQUIRE(dyn == nullptr || m->stu_mode == 1, FSTU_EARG, "fstu_decode_step: graph replay needs the recurrence (lds) STU state");
  FSTU_REQUIRE(m->layers && m->emb && m->final_norm_w && m->x && m->h && m->act && m->partial && m->logits,
               FSTU_ENULL, "fstu_decode_step: incomplete model descriptor");
  FSTU_REQUIRE(m->B >= 1 && m->B <= 2 * FSTU_MAX_DECODE_ROWS, FSTU_ESHAPE, "fstu_decode_step: batch %d outside 1..%d", m->B,
               2 * FSTU_MAX_DECODE_ROWS);
  FSTU_REQUIRE(m->n_layers >= 1 && m->ksplit_down >= 1 && pos >= 0, FSTU_EARG, "fstu_decode_step: bad layer count / split / pos");
  FSTU_REQUIRE(tok_stride >= 1, FSTU_EARG, "fstu_decode_step: tok_stride < 1");
  const int B = m->B, d = m->d, I = m->I, dt = m->dtype;
  const size_t esz = (dt == FSTU_BF16) ? 2 : 4;
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    if (L.kind == 0) {
      FSTU_REQUIRE(L.m_inputs_t, FSTU_ENULL, "fstu_decode_step: layer %d has no M_inputs", l);
      if (m->stu_mode == 0) {
        FSTU_REQUIRE(L.hist && L.filt && m->eo, FSTU_ENULL, "fstu_decode_step: layer %d has no history state", l);
        FSTU_REQUIRE(pos < m->hist_cap && pos < m->L, FSTU_EARG, "fstu_decode_step: position %d beyond history capacity %d / filter length %d", pos, m->hist_cap, m->L);
      } else {
        FSTU_REQUIRE(L.lds_a && L.lds_ce && L.lds_state && m->xp && m->y, FSTU_ENULL, "fstu_decode_step: layer %d has no recurrence state", l);
      }
    } else {
      FSTU_REQUIRE(L.w_qkv && L.w_proj && L.kring && L.vring && L.slopes && m->qkv && m->attn && m->y, FSTU_ENULL,
                   "fstu_decode_step: layer %d has no attention state", l);
    }
  }
  if (m->B > FSTU_MAX_DECODE_ROWS)
    return decode_step_wide(m, tok_in, tok_out, tok_stride, pos, temperature, top_k, top_p, do_sample, seed, step, dyn, stream);
  // x = embedding rows, h = norm(x) with the first layer's norm weight
  const bool chain = chain_ok(m, do_sample, dyn);
  if (chain && g_chain_prev)
    TIMED(PC_NORM, fstu_finish_embed_rmsnorm(m->best, tok_out, tok_stride, m->emb, m->x, m->layers[0].norm1_w, m->h, dyn, B, d,
                                             m->V, m->eps, stream));
  else
    TIMED(PC_NORM, fstu_embed_rmsnorm(tok_in, tok_stride, m->emb, m->x, m->layers[0].norm1_w, m->h, B, d, m->V, m->eps, dt,
                                      stream, dyn));
  // The residual stream starts in m->x.  Where a layer has packed gate/up weights, its MLP norm runs as the
  // prologue of the gate/up launch, which writes the updated residual to the other buffer (xc <-> xo swap).
  void* xc = m->x;
  void* xo = m->x2;
  const bool glu_bal = dt == FSTU_BF16 && m->glu_packed && fstu_glu_packed_supported(B, d, I);
  // Merged norms: the down projection leaves 4 split-K slices and the first projection of the NEXT layer adds them
  // to the residual stream and normalises it in its own prologue, so the add+norm launch between two layers is gone
  // (the one in front of the head stays).
  bool merge_norm = m->merge_norm && glu_bal && m->down_packed && m->x2 && m->stu_mode == 1 && d % 256 == 0 &&
                    (size_t)B * (d / 8) <= 1024 && I % 128 == 0 && I / 128 <= 96;
  for (int l = 0; l < m->n_layers && merge_norm; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    merge_norm = L.wp_gate && L.wp_up && L.wp_down && (L.kind == 0 || L.wp_qkv);
  }
  bool pending_slices = false;   // m->partial holds 4 slices of the previous layer's MLP output, not yet added
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    bool pending_y = false;   // m->y holds a sub-layer output not yet added to the residual stream
    if (L.kind == 0) {
      if (m->stu_mode == 0) {
        char* row = (char*)L.hist + (size_t)pos * d * esz;  // hist[:, pos, :] with row stride hist_cap*d
        TIMED(PC_PROJ, fstu_linear_decode(m->h, d, L.m_inputs_t, row, m->hist_cap * d, B, d, d, dt, stream));
        int ns = hist_nsplit(pos + 1, m->hist_nsplit_max);
        TIMED(PC_STU, fstu_stu_step_hist(L.hist, L.filt, m->eo, B, d, pos, m->hist_cap, m->L, ns, dt, stream));
        TIMED(PC_NORM, fstu_add_rmsnorm(xc, m->eo, 2, ns, m->single_branch, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
      } else {
        if (pending_slices) {
          TIMED(PC_STU, fstu_stu_res_inproj_step_dyn(xc, m->partial, 4, xo, L.norm1_w, m->eps, L.m_inputs_t, L.lds_state, L.lds_a,
                                                     L.lds_ce, L.lds_co, L.lds_ring, L.lds_fir, L.lds_fir ? m->lds_fir_taps : 0,
                                                     m->y, d, B, m->lds_S, d, d, stu_pos(pos), stu_dyn(dyn), dyn, stream));
          void* t = xc; xc = xo; xo = t;
          pending_slices = false;
        } else if (dt == FSTU_BF16 && d % 256 == 0) {
          TIMED(PC_STU, fstu_stu_inproj_step_dyn(m->h, d, L.m_inputs_t, L.lds_state, L.lds_a, L.lds_ce, L.lds_co, L.lds_ring, L.lds_fir,
                                                 L.lds_fir ? m->lds_fir_taps : 0, m->y, d, nullptr, B, m->lds_S, d, d, stu_pos(pos),
                                                 stu_dyn(dyn), dyn, stream));
        } else {
          TIMED(PC_PROJ, fstu_linear_decode(m->h, d, L.m_inputs_t, m->xp, d, B, d, d, dt, stream));
          TIMED(PC_STU, stu_step(L, m, stu_pos(pos), stu_dyn(dyn), dyn, stream));
        }
        pending_y = true;
      }
    } else {
      if (pending_slices) {
        TIMED(PC_PROJ, fstu_linear_packed_res(xc, m->partial, 4, xo, L.norm1_w, m->eps, L.wp_qkv, m->qkv, 3 * d, B, 3 * d, d,
                                              stream));
        void* t = xc; xc = xo; xo = t;
        pending_slices = false;
      } else if (glu_bal && L.wp_qkv)
        TIMED(PC_PROJ, fstu_linear_packed(m->h, d, nullptr, 0.f, L.wp_qkv, m->qkv, 3 * d, B, 3 * d, d, stream));
      else
        TIMED(PC_PROJ, fstu_linear_decode(m->h, d, L.w_qkv, m->qkv, 3 * d, B, 3 * d, d, dt, stream));
      TIMED(PC_SWA, fstu_swa_decode_impl(m->qkv, L.kring, L.vring, m->attn, L.slopes, B, m->n_heads, m->head_dim,
                                         m->kv_cap, pos, m->window, m->softcap, 1, dyn, dt, stream));
      TIMED(PC_PROJ, fstu_linear_decode(m->attn, d, L.w_proj, m->y, d, B, d, d, dt, stream));
      pending_y = true;
    }
    const void* next_w = (l + 1 < m->n_layers) ? m->layers[l + 1].norm1_w : m->final_norm_w;
    if (pending_y && glu_bal && m->x2 && L.wp_gate && L.wp_up) {
      // residual add + mlp_norm as the prologue of the balanced gate/up launch; the stream moves to the other buffer
      TIMED(PC_GLU, fstu_glu_packed_norm(xc, m->y, xo, L.mlp_norm_w, m->eps, L.wp_gate, L.wp_up, m->act, I, B, I, d, stream));
      void* t = xc; xc = xo; xo = t;
    } else {
      if (pending_y) TIMED(PC_NORM, fstu_add_rmsnorm(xc, m->y, 0, 1, 0, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
      if (glu_bal && L.wp_gate && L.wp_up)
        TIMED(PC_GLU, fstu_glu_packed(m->h, d, L.wp_gate, L.wp_up, m->act, I, B, I, d, stream));
      else
        TIMED(PC_GLU, fstu_glu_decode(m->h, d, L.w_gate, L.w_up, m->act, I, B, I, d, dt, stream));
    }
    if (merge_norm) {
      int nsl = 4;
      TIMED(PC_DOWN, fstu_down_packed_splitk(m->act, I, L.wp_down, m->partial, B, d, I, &nsl, stream));
      if (l + 1 == m->n_layers)   // the head reads normalised rows
        TIMED(PC_NORM, fstu_add_rmsnorm(xc, m->partial, 1, nsl, 0, next_w, m->h, B, d, m->eps, dt, stream));
      else
        pending_slices = true;
      continue;
    }
    int nsl = 16;
    if (glu_bal && m->down_packed && L.wp_down && d % 16 == 0 && I % 512 == 0 && I / 512 <= 64)
      TIMED(PC_DOWN, fstu_down_packed_splitk(m->act, I, L.wp_down, m->partial, B, d, I, &nsl, stream));
    else {
      nsl = m->ksplit_down;
      TIMED(PC_DOWN, fstu_linear_decode_splitk(m->act, I, L.w_down, m->partial, B, d, I, m->ksplit_down, dt, stream));
    }
    TIMED(PC_NORM, fstu_add_rmsnorm(xc, m->partial, 1, nsl, 0, next_w, m->h, B, d, m->eps, dt, stream));
  }
  // the head over the packed copy of the embedding where the model holds one: a workgroup keeps the activations in
  // registers for its whole share of the vocabulary and issues one atomic per row (768-d, 8 rows: 14.2 us against
  // 17.4 us for the row-major kernel, whose workgroups own 16 vocabulary rows each)
  const bool head_packed = dt == FSTU_BF16 && m->wp_emb && m->best && fstu_glu_packed_supported(B, d, m->V);
  if (!do_sample && m->best) {
    const int adv = (chain && g_chain_next) ? -1 : 1;   // < 0: the next step's first launch reduces the maxima
    if (head_packed) {
      TIMED(PC_HEAD, fstu_head_maxima_packed(m->h, d, m->wp_emb, m->logits, m->V, B, m->V, d, temperature, m->best, stream));
      if (adv >= 0) STEP(fstu_argmax_finish_launch(m->best, tok_out, tok_stride, B, dyn, adv, stream));
    } else {
      TIMED(PC_HEAD, fstu_head_argmax_dyn(m->h, d, m->emb, m->logits, m->V, B, m->V, d, temperature, m->best, tok_out, tok_stride, dyn,
                                          adv, dt, stream));
    }
  } else if (sample_spread_ok(m, do_sample, top_k)) {
    if (head_packed) TIMED(PC_HEAD, fstu_head_maxima_packed(m->h, d, m->wp_emb, m->logits, m->V, B, m->V, d, temperature, m->best, stream));
    else TIMED(PC_HEAD, fstu_head_maxima(m->h, d, m->emb, m->logits, m->V, B, m->V, d, temperature, m->best, dt, stream));
    TIMED(PC_SAMPLE, fstu_sample_topk_dyn(m->logits, m->V, m->best, m->samp_ws, tok_out, tok_stride, B, m->V, temperature, top_k, top_p,
                                          seed, step, m->row0, dyn, 1, stream));
  } else {
    TIMED(PC_HEAD, fstu_linear_decode(m->h, d, m->emb, m->logits, m->V, B, m->V, d, dt, stream));
    TIMED(PC_SAMPLE, fstu_sample_dyn(m->logits, tok_out, tok_stride, B, m->V, temperature, top_k, top_p, do_sample, seed, step, m->row0, dyn, dt, stream));
    if (dyn) STEP(fstu_advance_dyn(dyn, stream));
  }
  return FSTU_OK;
}

extern "C" int fstu_decode_step(const fstu_model_desc* m, const int64_t* tok_in, int64_t* tok_out, int64_t tok_stride,
                                int pos, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                                int step, void* stream) {
  return decode_step_impl(m, tok_in, tok_out, tok_stride, pos, temperature, top_k, top_p, do_sample, seed, step, nullptr,
                          stream);
}

// ---------------------------------------------------------------- one step as a replayable HIP graph
struct fstu_graph {
  hipGraph_t graph[2];       // one per parity of the position (the second is null when the model has no STU state)
  hipGraphExec_t exec[2];
  long long next_pos;        // position the next launch will process first
  int nsteps;                // decode steps per launch
  bool baked;                // the STU launches carry the parity of their position as an argument
};

extern "C" int fstu_decode_graph_create(const fstu_model_desc* m, int64_t* tokens, int64_t tok_stride, int* dyn, int pos0,
                                        int nsteps, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                                        void* stream, void** graph_out) {
  FSTU_REQUIRE(m && tokens && dyn && graph_out && stream, FSTU_ENULL, "fstu_decode_graph_create: null pointer (a non-default stream is required)");
  FSTU_REQUIRE(pos0 >= 0 && nsteps >= 1 && nsteps <= 64, FSTU_EARG, "fstu_decode_graph_create: pos0=%d nsteps=%d (1..64)", pos0, nsteps);
  hipStream_t s = (hipStream_t)stream;
  // One graph per parity of the first position: the STU launches carry their parity as an argument.  A graph of an
  // even number of steps always starts on the parity of pos0, so the other one is not captured.
  const bool baked = m->stu_mode == 1;
  fstu_graph* h = new fstu_graph{{nullptr, nullptr}, {nullptr, nullptr}, pos0, nsteps, baked};
  for (int par = 0; par < 2; ++par) {
    if (!baked && par == 1) break;
    if (baked && (nsteps & 1) == 0 && par != (pos0 & 1)) continue;
    hipError_t e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) { fstu_decode_graph_destroy(h); fstu_set_error("fstu_decode_graph_create: begin capture: %s", hipGetErrorString(e)); return (int)e; }
    int rc = 0;
    for (int st = 0; st < nsteps && rc == 0; ++st) {
      g_stu_parity = baked ? ((par + st) & 1) : -1;
      g_chain_prev = st > 0;
      g_chain_next = st + 1 < nsteps;
      rc = decode_step_impl(m, tokens, tokens + 1, tok_stride, 0, temperature, top_k, top_p, do_sample, seed, 0, dyn, stream);
    }
    g_stu_parity = -1;
    g_chain_prev = g_chain_next = false;
    e = hipStreamEndCapture(s, &h->graph[par]);
    if (rc != 0) { fstu_decode_graph_destroy(h); return rc; }
    if (e != hipSuccess) { fstu_decode_graph_destroy(h); fstu_set_error("fstu_decode_graph_create: end capture: %s", hipGetErrorString(e)); return (int)e; }
    e = hipGraphInstantiate(&h->exec[par], h->graph[par], nullptr, nullptr, 0);
    if (e != hipSuccess) { fstu_decode_graph_destroy(h); fstu_set_error("fstu_decode_graph_create: instantiate: %s", hipGetErrorString(e)); return (int)e; }
  }
  *graph_out = h;
  return FSTU_OK;
}

extern "C" int fstu_decode_graph_launch(void* graph, void* stream) {
  FSTU_REQUIRE(graph, FSTU_ENULL, "fstu_decode_graph_launch: null graph");
  fstu_graph* h = (fstu_graph*)graph;
  int par = (int)(h->next_pos & 1);
  if (!h->exec[par]) par ^= 1;   // position-independent graph, or an even number of steps per graph
  hipError_t e = hipGraphLaunch(h->exec[par], (hipStream_t)stream);
  if (e != hipSuccess) { fstu_set_error("fstu_decode_graph_launch: %s", hipGetErrorString(e)); return (int)e; }
  h->next_pos += h->nsteps;
  return FSTU_OK;
}

extern "C" int fstu_decode_graph_seek(void* graph, long long next_pos) {
  FSTU_REQUIRE(graph && next_pos >= 0, FSTU_EARG, "fstu_decode_graph_seek: null graph or negative position");
  fstu_graph* h = (fstu_graph*)graph;
  // with the parity of the position baked into the STU launches, a graph of an even number of steps exists for one
  // parity of its first position only
  FSTU_REQUIRE(!h->baked || h->exec[next_pos & 1], FSTU_EARG,
               "fstu_decode_graph_seek: this %d-step graph was captured for positions of the other parity", h->nsteps);
  h->next_pos = next_pos;
  return FSTU_OK;
}

extern "C" int fstu_decode_graph_destroy(void* graph) {
  if (!graph) return FSTU_OK;
  fstu_graph* h = (fstu_graph*)graph;
  for (int par = 0; par < 2; ++par) {
    if (h->exec[par]) (void)hipGraphExecDestroy(h->exec[par]);
    if (h->graph[par]) (void)hipGraphDestroy(h->graph[par]);
  }
  delete h;
  return FSTU_OK;
}
