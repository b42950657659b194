"""Decode engine behind FlashSTU.generate(): prefill through the module path,
then one C-ABI call per token (fstu_decode_step) that launches the fused kernel
sequence for the whole layer stack against preallocated state and workspaces,
or the same step captured once as a HIP graph and replayed per token.

The token buffer (B, max_length) lives on the GPU for the whole loop; each step
reads column pos and writes column pos+1, so the host never sees a token until
generate() returns (reference loop: flash_stu/model.py:245-302, which re-allocates
the sequence with torch.cat every step).

The decode kernels take at most 16 activation rows; a larger batch runs as
consecutive row chunks of 16 against the same weights and batch-first state.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from . import _hip
from .layers.attention_layer import AttentionLayer
from .layers.stu_layer import STULayer

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


class LayerDesc(ctypes.Structure):
    _fields_ = [("kind", _i), ("norm1_w", _vp), ("mlp_norm_w", _vp), ("w_gate", _vp), ("w_up", _vp), ("w_down", _vp),
                ("m_inputs_t", _vp), ("filt", _vp), ("hist", _vp), ("lds_a", _vp), ("lds_ce", _vp), ("lds_co", _vp), ("lds_state", _vp), ("lds_ring", _vp), ("lds_fir", _vp), ("lds_ocache", _vp),
                ("w_qkv", _vp), ("w_proj", _vp), ("kring", _vp), ("vring", _vp), ("slopes", _vp),
                ("wp_gate", _vp), ("wp_up", _vp), ("wp_down", _vp), ("wp_m_inputs", _vp), ("wp_qkv", _vp),
                ("wp_proj", _vp)]


class ModelDesc(ctypes.Structure):
    _fields_ = [("dtype", _i), ("B", _i), ("d", _i), ("I", _i), ("V", _i), ("n_layers", _i), ("n_heads", _i),
                ("head_dim", _i), ("window", _i), ("kv_cap", _i), ("L", _i), ("hist_cap", _i), ("stu_mode", _i),
                ("lds_S", _i), ("lds_fir_taps", _i), ("single_branch", _i), ("ksplit_down", _i), ("hist_nsplit_max", _i), ("row0", _i),
                ("eps", _f), ("softcap", _f), ("emb", _vp), ("final_norm_w", _vp), ("layers", ctypes.POINTER(LayerDesc)),
                ("x", _vp), ("h", _vp), ("qkv", _vp), ("attn", _vp), ("act", _vp), ("xp", _vp), ("y", _vp),
                ("partial", _vp), ("eo", _vp), ("logits", _vp), ("best", _vp), ("samp_ws", _vp),
                ("wp_emb", _vp), ("x2", _vp), ("glu_packed", _i), ("down_packed", _i), ("merge_norm", _i)]


def pick_ksplit_down(I: int) -> int:
    """K split of the down projection: enough waves to fill 256 CUs while every
    slice still divides into the 64-wide k steps of the MFMA kernel."""
    for ks in (12, 16, 8, 6, 4, 3, 2):
        if I % (ks * 256) == 0:
            return ks
    for ks in (8, 4, 2):
        if I % (ks * 64) == 0:
            return ks
    return 1


class _Chunk:
    """Descriptor, workspaces and graph handle of one chunk of at most 16 batch rows."""

    def __init__(self, b0: int, b1: int):
        self.b0, self.b1 = b0, b1
        self.keep: List[torch.Tensor] = []
        self.arr = None
        self.desc: Optional[ModelDesc] = None
        self.logits: Optional[torch.Tensor] = None
        self.graphs = {}            # steps per graph -> handle
        self.dyn: Optional[torch.Tensor] = None
        self.stream = None


class DecodeEngine:
    HIST_NSPLIT_MAX = 16

    @staticmethod
    def supports(cfg) -> bool:
        """The one-call decode step covers approx-mode STU layers without the sandwich and bias-free linears;
        other variants decode through the layers' own state (FlashSTU.generate picks the loop)."""
        if cfg.use_hankel_L and cfg.resolved_stu_decode_mode() == "lds":
            return False     # single-branch filters on the recurrence state: the odd lags read the other bank
        return bool(cfg.use_approx) and not cfg.stu_enable_mlp_sandwich and not cfg.bias

    def __init__(self, model):
        cfg = model.config
        if not self.supports(cfg):
            raise NotImplementedError("the fused decode engine covers use_approx=True without the STU sandwich and "
                                      "without biases; FlashSTU.generate falls back to the per-layer state loop")
        self.model = model
        self.cfg = cfg
        self.lib = _hip.load()
        self.chunks: List[_Chunk] = []
        self._packed = {}
        self._gstream = None
        self._gstreams = []

    # ------------------------------------------------------------------
    def _pack(self, w: torch.Tensor) -> torch.Tensor:
        """MFMA-fragment-ordered copy of an (N,K) bf16 weight, rebuilt only when the weight changes."""
        key = w.data_ptr()
        hit = self._packed.get(key)
        if hit is None or hit[0] != w._version:
            hit = (w._version, _hip.pack_rows(w))
            self._packed[key] = hit
        return hit[1]

    @property
    def desc(self) -> ModelDesc:
        """Descriptor of the first row chunk (the whole batch when B <= 16)."""
        return self.chunks[0].desc

    @property
    def logits(self) -> torch.Tensor:
        """(B,V) logits of the last eager step."""
        return self.chunks[0].logits if len(self.chunks) == 1 else torch.cat([c.logits for c in self.chunks], 0)

    def _build(self, caches, B: int, total_len: int):
        cfg = self.cfg
        d = cfg.n_embd
        mode = cfg.resolved_stu_decode_mode()
        caches = list(caches)
        if mode != "lds":                      # history buffers must hold the whole generation
            for i, layer in enumerate(self.model.layers):
                if isinstance(layer, STULayer):
                    hist, state, pos = caches[i]
                    if hist.shape[1] < total_len:
                        bigger = hist.new_zeros(B, total_len, d)
                        bigger[:, : hist.shape[1]] = hist
                        caches[i] = (bigger, state, pos)
        self.graph_end()
        self.chunks = []
        R = _hip.MAX_DECODE_ROWS
        # Rows are stepped in chunks of up to 16 (the width of the skinny decode kernels), each chunk re-reading the
        # weights.  A chunk of 17..32 rows instead runs its MLP, nearly all of the weight bytes, once over all rows on the
        # tiled GEMM kernel (bf16, recurrence STU state).
        wide = (cfg.torch_dtype == torch.bfloat16 and mode == "lds" and d % 256 == 0 and (d * cfg.mlp_scale) % 64 == 0)
        b0 = 0
        while b0 < B:
            rows = min(B - b0, 2 * R if (wide and B - b0 > R) else R)
            ch = _Chunk(b0, b0 + rows)
            self._build_chunk(ch, caches)
            self.chunks.append(ch)
            b0 += rows
        return tuple(caches)

    def _build_chunk(self, ch: _Chunk, caches):
        model, cfg = self.model, self.cfg
        dev = model.lm_head.weight.device
        dt = cfg.torch_dtype
        d, I, V = cfg.n_embd, cfg.n_embd * cfg.mlp_scale, cfg.vocab_size
        mode = cfg.resolved_stu_decode_mode()
        b0, b1 = ch.b0, ch.b1
        B = b1 - b0
        keep = ch.keep.append
        n = len(model.layers)
        arr = (LayerDesc * n)()
        hist_cap = 0
        fir_taps = 0
        for i, layer in enumerate(model.layers):
            ld = arr[i]
            ld.w_gate = layer.mlp.gate_proj.weight.data_ptr()
            ld.w_up = layer.mlp.up_proj.weight.data_ptr()
            ld.w_down = layer.mlp.down_proj.weight.data_ptr()
            ld.mlp_norm_w = layer.mlp_norm.weight.data_ptr()
            if isinstance(layer, STULayer):
                stu = layer.stu
                ld.kind = 0
                ld.norm1_w = layer.stu_norm.weight.data_ptr()
                mit = stu.m_inputs_t()
                keep(mit)
                ld.m_inputs_t = mit.data_ptr()
                hist, state, pos = caches[i]
                if mode == "lds":
                    a, ce, co = stu.lds_params()
                    st = state[b0:b1]
                    keep(a), keep(ce), keep(co), keep(st)
                    ld.lds_a, ld.lds_ce, ld.lds_co, ld.lds_state = a.data_ptr(), ce.data_ptr(), co.data_ptr(), st.data_ptr()
                    fir = stu.lds_fir()
                    if fir is not None and hist.shape[1] == fir.shape[0]:
                        ring = hist[b0:b1]       # in lds mode the history slot of the cache entry is the ring of the last inputs
                        keep(fir), keep(ring)
                        ld.lds_ring, ld.lds_fir = ring.data_ptr(), fir.data_ptr()
                        fir_taps = fir.shape[0]
                    if B > _hip.MAX_DECODE_ROWS and dt == torch.bfloat16 and not cfg.use_hankel_L:
                        # 17..32 rows: the odd-lag sum is handed from step to step, so a step reads one bank only;
                        # primed here for the first decode position from the state and ring the prompt left
                        oc = _hip.stu_step_lds_prime(st, a, co, int(pos[0]) - 1, dt,
                                                     ring=hist[b0:b1] if ld.lds_ring else None, fir=fir if ld.lds_ring else None)
                        keep(oc)
                        ld.lds_ocache = oc.data_ptr()
                else:
                    hs = hist[b0:b1]
                    if hist_cap and hs.shape[1] != hist_cap:
                        raise RuntimeError("STU histories must share one capacity")
                    hist_cap = hs.shape[1]
                    filt = stu.effective_filter()
                    keep(filt), keep(hs)
                    ld.filt, ld.hist = filt.data_ptr(), hs.data_ptr()
            elif isinstance(layer, AttentionLayer):
                att = layer.attn
                ld.kind = 1
                ld.norm1_w = layer.attn_norm.weight.data_ptr()
                ld.w_qkv = att.c_attn.weight.data_ptr()
                ld.w_proj = att.c_proj.weight.data_ptr()
                kr, vr, pos = caches[i]
                kr, vr = kr[b0:b1], vr[b0:b1]
                keep(kr), keep(vr)
                ld.kring, ld.vring = kr.data_ptr(), vr.data_ptr()
                ld.slopes = att.alibi_slopes.data_ptr()
            else:
                raise TypeError(type(layer))
        m = ModelDesc()
        m.dtype = _hip.FSTU_BF16 if dt == torch.bfloat16 else _hip.FSTU_F32
        m.B, m.d, m.I, m.V, m.n_layers = B, d, I, V, n
        m.n_heads, m.head_dim = cfg.n_heads, d // cfg.n_heads
        m.window, m.kv_cap = cfg.window_left, cfg.window_left + 1
        m.L, m.hist_cap = cfg.seq_len, hist_cap
        m.stu_mode = 1 if mode == "lds" else 0
        m.lds_S = cfg.stu_lds_state_dim
        m.lds_fir_taps = fir_taps
        m.single_branch = int(cfg.use_hankel_L)
        m.ksplit_down = pick_ksplit_down(I) if dt == torch.bfloat16 else min(8, max(1, I // 512))
        m.hist_nsplit_max = self.HIST_NSPLIT_MAX
        m.row0 = b0
        m.eps, m.softcap = float(cfg.rms_norm_eps), float(cfg.softcap or 0.0)
        m.emb = model.lm_head.weight.data_ptr()
        m.final_norm_w = model.norm.weight.data_ptr()
        m.layers = ctypes.cast(arr, ctypes.POINTER(LayerDesc))

        def buf(*shape, dtype=dt):
            t = torch.zeros(*shape, dtype=dtype, device=dev)
            keep(t)
            return t
        ch.logits = buf(B, V)
        m.x, m.h = buf(B, d).data_ptr(), buf(B, d).data_ptr()
        m.qkv, m.attn = buf(B, 3 * d).data_ptr(), buf(B, d).data_ptr()
        m.act, m.xp, m.y = buf(B, I).data_ptr(), buf(B, d).data_ptr(), buf(B, d).data_ptr()
        m.partial = buf(max(m.ksplit_down, 16), B, d, dtype=torch.float32).data_ptr()
        m.eo = buf(self.HIST_NSPLIT_MAX, 2, B, d, dtype=torch.float32).data_ptr()
        m.logits = ch.logits.data_ptr()
        m.best = buf(32 * 64, dtype=torch.int64).data_ptr()
        m.samp_ws = buf((int(self.lib.fstu_sample_ws_bytes()) + 7) // 8, dtype=torch.int64).data_ptr()
        if dt == torch.bfloat16 and self.lib.fstu_glu_packed_supported(B, d, I):
            # gate/up projection over packed weights, one workgroup per CU with equal bytes each
            for i, layer in enumerate(model.layers):
                arr[i].wp_gate = self._pack(layer.mlp.gate_proj.weight).data_ptr()
                arr[i].wp_up = self._pack(layer.mlp.up_proj.weight).data_ptr()
            m.glu_packed = 1
            if I % 512 == 0 and d % 16 == 0:
                for i, layer in enumerate(model.layers):
                    arr[i].wp_down = self._pack(layer.mlp.down_proj.weight).data_ptr()
                m.down_packed = 1
            if B * (d + 8) * 2 <= 96 * 1024:
                m.x2 = buf(B, d).data_ptr()     # second residual buffer: the MLP norm runs as the gate/up prologue
                if mode == "lds" and d % 256 == 0 and m.down_packed and B * (d // 8) <= 1024 and I % 128 == 0:
                    # the add+norm between two layers runs as the prologue of the next layer's first projection
                    # (the down projection leaves 4 split-K slices for it): one launch less per layer
                    for i, layer in enumerate(model.layers):
                        if isinstance(layer, AttentionLayer):
                            arr[i].wp_qkv = self._pack(layer.attn.c_attn.weight).data_ptr()
                    m.merge_norm = 1
        if dt == torch.bfloat16 and self.lib.fstu_mlp_packed_rows32_supported(B, d, I):
            # 17..32 rows: the MLP streams packed weights as two row tiles per weight fragment
            for i, layer in enumerate(model.layers):
                arr[i].wp_gate = self._pack(layer.mlp.gate_proj.weight).data_ptr()
                arr[i].wp_up = self._pack(layer.mlp.up_proj.weight).data_ptr()
                arr[i].wp_down = self._pack(layer.mlp.down_proj.weight).data_ptr()
                if isinstance(layer, AttentionLayer):
                    arr[i].wp_qkv = self._pack(layer.attn.c_attn.weight).data_ptr()
                    arr[i].wp_proj = self._pack(layer.attn.c_proj.weight).data_ptr()
                elif mode == "lds":
                    arr[i].wp_m_inputs = self._pack(layer.stu.m_inputs_t()).data_ptr()
        if dt == torch.bfloat16 and self.lib.fstu_glu_packed_supported(min(B, _hip.MAX_DECODE_ROWS), d, V):
            m.wp_emb = self._pack(model.lm_head.weight).data_ptr()      # the head streams a packed copy of the embedding
        ch.arr, ch.desc = arr, m
        if B > _hip.MAX_DECODE_ROWS:
            # first use of the tiled kernels outside any graph capture (their launch set-up raises an LDS limit once)
            wx = torch.zeros(B, 64, dtype=dt, device=dev)
            ww = torch.zeros(8, 64, dtype=dt, device=dev)
            _hip.gemm(wx, ww, up_weight=ww)
            _hip.gemm_splitk(wx, ww, 1)

    # ------------------------------------------------------------------ eager step
    def step(self, tokens: torch.Tensor, pos: int, temperature, top_k, top_p, do_sample, seed, step_idx):
        """Feeds tokens[:, pos], writes the sampled id to tokens[:, pos+1]."""
        stride = tokens.stride(0)
        for ch in self.chunks:
            base = tokens.data_ptr() + 8 * (ch.b0 * stride + pos)
            rc = self.lib.fstu_decode_step(ctypes.byref(ch.desc), base, base + 8, stride, pos, float(temperature),
                                           int(top_k) if top_k else 0, float(top_p) if top_p else 0.0,
                                           int(bool(do_sample)), int(seed) & ((1 << 64) - 1), int(step_idx),
                                           torch.cuda.current_stream().cuda_stream)
            _hip._check(rc, "fstu_decode_step")

    # ------------------------------------------------------------------ graph replay
    def graph_supported(self) -> bool:
        return self.cfg.resolved_stu_decode_mode() == "lds"

    GRAPH_STEPS = 8     # decode steps per graph launch in generate() (the launch of a graph costs several microseconds)

    def graph_begin(self, tokens: torch.Tensor, pos: int, step_idx: int, temperature, top_k, top_p, do_sample, seed,
                    steps_per_graph: int = 1, keep: bool = False):
        """Captures steps_per_graph decode steps per row chunk as a HIP graph, each chunk on a side stream of its own: the
        chunks are independent (own workspaces, state rows and device-side position), so their graphs run concurrently
        and the second chunk finds the layer's weights, which the first has just streamed, in the Infinity Cache.  Each
        graph_step() then runs steps_per_graph decode steps: each feeds tokens[:, pos], writes tokens[:, pos+1] and
        advances pos on the device.  `pos` is the position the first launch of THIS graph will process.  keep=True adds
        the graph to those already captured (same tokens, sampling arguments and device-side counters) instead of
        replacing them: a run can then mix long graphs with single-step ones (graph_step(n), graph_seek)."""
        if not keep:
            self.graph_end()
        n = int(steps_per_graph)
        self.graph_steps = n
        n_streams = len(self.chunks)
        if not self._gstreams:
            self._gstreams = [torch.cuda.Stream(device=tokens.device) for _ in range(n_streams)]
        stride = tokens.stride(0)
        for ch in self.chunks:
            if ch.dyn is None:
                ch.dyn = torch.tensor([pos, step_idx], dtype=torch.int32, device=tokens.device)
        for st in self._gstreams:
            st.wait_stream(torch.cuda.current_stream())
        for i, ch in enumerate(self.chunks):
            handle = _vp()
            ch.stream = self._gstreams[i % len(self._gstreams)]
            rc = self.lib.fstu_decode_graph_create(ctypes.byref(ch.desc), tokens.data_ptr() + 8 * ch.b0 * stride, stride,
                                                   ch.dyn.data_ptr(), int(pos), n, float(temperature),
                                                   int(top_k) if top_k else 0,
                                                   float(top_p) if top_p else 0.0, int(bool(do_sample)),
                                                   int(seed) & ((1 << 64) - 1), ch.stream.cuda_stream,
                                                   ctypes.byref(handle))
            _hip._check(rc, "fstu_decode_graph_create")
            ch.graphs[n] = handle
        self._graph_tokens = tokens

    def graph_step(self, steps_per_graph: Optional[int] = None):
        n = self.graph_steps if steps_per_graph is None else int(steps_per_graph)
        for ch in self.chunks:
            _hip._check(self.lib.fstu_decode_graph_launch(ch.graphs[n], ch.stream.cuda_stream), "fstu_decode_graph_launch")

    def graph_seek(self, steps_per_graph: int, pos: int):
        """Tells the graph of that length which position its next launch will process (needed after graphs of another
        length have advanced the device-side position in between)."""
        for ch in self.chunks:
            _hip._check(self.lib.fstu_decode_graph_seek(ch.graphs[int(steps_per_graph)], int(pos)), "fstu_decode_graph_seek")

    def graph_sync(self):
        """Blocks until every chunk's replay stream has drained."""
        for st in self._gstreams:
            st.synchronize()

    def graph_end(self):
        live = [ch for ch in self.chunks if ch.graphs]
        if live:
            for st in self._gstreams:
                torch.cuda.current_stream().wait_stream(st)
                st.synchronize()
            for ch in live:
                for handle in ch.graphs.values():
                    self.lib.fstu_decode_graph_destroy(handle)
                ch.graphs = {}
        for ch in self.chunks:
            ch.dyn = None
        self._gstreams = []

    # ------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor, total_len: int):
        """Runs the prompt through the module path with caches, returns the
        logits of the last position (B,V) and prepares the step descriptors."""
        model = self.model
        B, P = input_ids.shape
        x = model._embed(input_ids.contiguous())
        x, caches = model._run_layers(x, None, True, None)
        xn = model.norm(x[:, -1:, :].contiguous())
        logits = model._head(xn)[:, 0, :].contiguous()
        self.caches = self._build(caches, B, total_len)
        return logits

    @torch.no_grad()
    def generate(self, input_ids: torch.Tensor, n_new: int, temperature=1.0, top_k=None, top_p=None, do_sample=True,
                 seed: int = 0, return_logits: bool = False, use_graph: bool = True):
        if not input_ids.is_cuda:
            raise _hip.FlashSTUHipError("input_ids must be on the GPU: this model has no CPU path")
        B, P = input_ids.shape
        total = P + n_new
        if total > self.cfg.seq_len:
            # the history ends there, and the recurrence state would carry a tail the filters (zero from lag seq_len
            # on) do not have; FlashSTU.generate routes such calls to the recompute loop
            raise ValueError(f"stateful decode needs prompt+new tokens ({total}) <= seq_len ({self.cfg.seq_len})")
        tokens = torch.zeros(B, total, dtype=torch.int64, device=input_ids.device)
        tokens[:, :P] = input_ids
        logits = self.prefill(input_ids, total)
        _hip.sample(logits, tokens[:, P], temperature, top_k, top_p, do_sample, seed, 0)
        all_logits = [logits.clone()] if return_logits else None
        if use_graph and not return_logits and self.graph_supported() and n_new > 2:
            todo, pos, S = n_new - 1, P, self.GRAPH_STEPS
            try:
                if todo >= 4 * S:       # long runs: S steps per graph launch, the remainder one by one
                    self.graph_begin(tokens, pos, pos - P + 1, temperature, top_k, top_p, do_sample, seed, steps_per_graph=S)
                    for _ in range(todo // S):
                        self.graph_step()
                    pos += (todo // S) * S
                    todo -= (todo // S) * S
                if todo > 0:
                    self.graph_begin(tokens, pos, pos - P + 1, temperature, top_k, top_p, do_sample, seed)
                    for _ in range(todo):
                        self.graph_step()
            finally:
                self.graph_end()
            return tokens
        for s in range(1, n_new):
            self.step(tokens, P + s - 1, temperature, top_k, top_p, do_sample, seed, s)
            if return_logits:
                all_logits.append(self.logits.clone())
        return (tokens, torch.stack(all_logits, 1)) if return_logits else tokens
