// Host-side driver of one decode step: the launch sequence over the layer
// stack, with every residual add fused into the RMSNorm that follows it.
#include "fstu_common.h"

#define STEP(call)          \
  do {                      \
    int rc__ = (call);      \
    if (rc__ != 0) return rc__; \
  } while (0)

static int hist_nsplit(int nlags, int maxsplit) {
  int n = nlags / 64;
  if (n < 1) n = 1;
  if (n > 16) n = 16;
  if (n > maxsplit) n = maxsplit;
  return n;
}

extern "C" int fstu_decode_step(const fstu_model_desc* m, const int64_t* tok_in, int64_t* tok_out, int64_t tok_stride,
                                int pos, float temperature, int top_k, float top_p, int do_sample, uint64_t seed,
                                int step, void* stream) {
  FSTU_REQUIRE(m && tok_in && tok_out, FSTU_ENULL, "fstu_decode_step: null pointer");
  FSTU_REQUIRE(m->layers && m->emb && m->final_norm_w && m->x && m->h && m->act && m->partial && m->logits,
               FSTU_ENULL, "fstu_decode_step: incomplete model descriptor");
  FSTU_REQUIRE(m->B >= 1 && m->B <= FSTU_MAX_DECODE_ROWS, FSTU_ESHAPE, "fstu_decode_step: batch %d outside 1..%d", m->B,
               FSTU_MAX_DECODE_ROWS);
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
  STEP(fstu_embed_strided(tok_in, tok_stride, m->emb, m->x, B, d, m->V, dt, stream));
  // h = norm(x) with the first layer's norm weight
  STEP(fstu_add_rmsnorm(m->x, nullptr, 0, 1, 0, m->layers[0].norm1_w, m->h, B, d, m->eps, dt, stream));
  for (int l = 0; l < m->n_layers; ++l) {
    const fstu_layer_desc& L = m->layers[l];
    if (L.kind == 0) {
      if (m->stu_mode == 0) {
        char* row = (char*)L.hist + (size_t)pos * d * esz;  // hist[:, pos, :] with row stride hist_cap*d
        STEP(fstu_linear_decode(m->h, d, L.m_inputs_t, row, m->hist_cap * d, B, d, d, dt, stream));
        int ns = hist_nsplit(pos + 1, m->hist_nsplit_max);
        STEP(fstu_stu_step_hist(L.hist, L.filt, m->eo, B, d, pos, m->hist_cap, m->L, ns, dt, stream));
        STEP(fstu_add_rmsnorm(m->x, m->eo, 2, ns, m->single_branch, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
      } else {
        STEP(fstu_linear_decode(m->h, d, L.m_inputs_t, m->xp, d, B, d, d, dt, stream));
        STEP(fstu_stu_step_lds(L.lds_state, m->xp, d, L.lds_a, L.lds_ce, m->y, d, B, m->lds_S, d, pos, dt, stream));
        STEP(fstu_add_rmsnorm(m->x, m->y, 0, 1, 0, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
      }
    } else {
      STEP(fstu_linear_decode(m->h, d, L.w_qkv, m->qkv, 3 * d, B, 3 * d, d, dt, stream));
      STEP(fstu_kv_append(m->qkv, L.kring, L.vring, B, m->n_heads, m->head_dim, m->kv_cap, pos, dt, stream));
      STEP(fstu_swa_decode(m->qkv, L.kring, L.vring, m->attn, L.slopes, B, m->n_heads, m->head_dim, m->kv_cap, pos,
                           m->window, m->softcap, dt, stream));
      STEP(fstu_linear_decode(m->attn, d, L.w_proj, m->y, d, B, d, d, dt, stream));
      STEP(fstu_add_rmsnorm(m->x, m->y, 0, 1, 0, L.mlp_norm_w, m->h, B, d, m->eps, dt, stream));
    }
    STEP(fstu_glu_decode(m->h, d, L.w_gate, L.w_up, m->act, I, B, I, d, dt, stream));
    STEP(fstu_linear_decode_splitk(m->act, I, L.w_down, m->partial, B, d, I, m->ksplit_down, dt, stream));
    const void* next_w = (l + 1 < m->n_layers) ? m->layers[l + 1].norm1_w : m->final_norm_w;
    STEP(fstu_add_rmsnorm(m->x, m->partial, 1, m->ksplit_down, 0, next_w, m->h, B, d, m->eps, dt, stream));
  }
  STEP(fstu_linear_decode(m->h, d, m->emb, m->logits, m->V, B, m->V, d, dt, stream));
  STEP(fstu_sample(m->logits, tok_out, tok_stride, B, m->V, temperature, top_k, top_p, do_sample, seed, step, dt, stream));
  return FSTU_OK;
}
