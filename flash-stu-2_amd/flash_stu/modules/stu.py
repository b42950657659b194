"""Spectral Transform Unit (reference: flash_stu/modules/stu.py:12-120).

Same parameters and forward semantics as the reference module; in addition the
module can carry decode state so that one token per call reproduces what the
reference obtains by re-running the whole sequence:

  history mode  the projected inputs x_proj of every past position are kept and
                the causal convolution is evaluated at the newest position by
                the HIP history kernel (exact; fp32 parity mode);
  lds mode      the even-lag effective filter is distilled into S real modes
                per channel and two parity banks of recurrence state replace
                the history (bounded state; bf16 performance mode).

State tuples are batch-first tensors: (hist (B,cap,d), state (B,2,S,d) fp32, pos (B,) int64 on the host); in lds mode
the history slot holds the ring of the last stu_lds_fir_taps projected inputs (B,R,d), or is empty.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn

from .. import _hip
from ..utils.lds_fit import check_lds_fit, fit_even_lag_lds


FFT_MIN_T = 32     # shorter inputs take the time-domain kernel (a 64-point transform would be mostly padding)


class STU(nn.Module):
    def __init__(self, config, phi: torch.Tensor, n: int, feature_dim: Optional[int] = None) -> None:
        super().__init__()
        self.config = config
        self.register_buffer("phi", phi, persistent=False)
        self.n = n
        self.K = config.num_eigh
        self.d_in = feature_dim if feature_dim is not None else config.n_embd
        self.d_out = self.d_in
        self.use_hankel_L = config.use_hankel_L
        self.use_approx = config.use_approx
        dt = config.torch_dtype
        if self.use_approx:
            self.M_inputs = nn.Parameter(torch.empty(self.d_in, self.d_out, dtype=dt))
            self.M_filters = nn.Parameter(torch.empty(self.K, self.d_in, dtype=dt))
        else:
            self.M_phi_plus = nn.Parameter(torch.empty(self.K, self.d_in, self.d_out, dtype=dt))
            if not self.use_hankel_L:
                self.M_phi_minus = nn.Parameter(torch.empty(self.K, self.d_in, self.d_out, dtype=dt))
        # channel tiling (stu.py:123-191): diagonal blocks of M_inputs only, i.e. M_inputs with every entry outside
        # the tile_size x tile_size diagonal blocks dropped; the convolution itself is per channel either way
        self.tile_size = min(config.d_in_tile or self.d_in, config.d_out_tile or self.d_in)
        if self.tile_size < self.d_in and not self.use_approx:
            raise NotImplementedError("Tiling only supported for use_approx=True")
        self._derived = {}

    # ---- tensors derived from the parameters, rebuilt when a parameter changes
    def _cached(self, key, params, build):
        ver = tuple((p._version, p.data_ptr()) for p in params)
        hit = self._derived.get(key)
        if hit is None or hit[0] != ver:
            hit = (ver, build())
            self._derived[key] = hit
        return hit[1]

    def decode_mode(self) -> str:
        mode = self.config.resolved_stu_decode_mode()
        if mode == "lds" and self.use_approx and self.use_hankel_L and self.phi.shape[0] % 2 != 0:
            return "history"     # the single-branch recurrence needs equally long even- and odd-lag halves
        return mode

    def _exact_lds_ok(self) -> bool:
        """Exact mode can decode on the recurrence state when asked for explicitly (stu_decode_mode='lds'), the
        filter length is even (equal pole grids for the even and odd lags) and K fits the bank kernel."""
        return (not self.use_approx and self.decode_mode() == "lds" and self.phi.shape[0] % 2 == 0 and self.K <= 32)

    def effective_filter(self) -> torch.Tensor:
        """phi_proj = phi @ M_filters, (L,d) in the model dtype (stu.py:88).  On the GPU the general contraction
        kernel; the host-side filter fit (lds_params / lds_fir in float64) may ask for it before the module has been
        moved to the GPU, and then it is a host matmul like the rest of that fit."""
        def build():
            if self.phi.is_cuda:
                return _hip.gemm_any(self.phi, self.M_filters.t())
            return torch.matmul(self.phi, self.M_filters).contiguous()
        return self._cached("filt", (self.phi, self.M_filters), build)

    def filter_spectrum(self, n: int) -> torch.Tensor:
        """Spectra of the convolution filters for transform length n, (d,n,2) fp32 in approx mode, (K,n,2) in
        exact mode (the reference keeps its own phi_fft the same way, stu.py:43-53).  One length is kept."""
        src = self.effective_filter() if self.use_approx else self.phi
        params = (self.phi, self.M_filters) if self.use_approx else (self.phi,)
        hit = self._derived.get("spec")
        if hit is not None and hit[1].shape[1] != n:
            self._derived.pop("spec")
        return self._cached("spec", params, lambda: _hip.stu_fft_filter(src, n, single_branch=self.use_hankel_L))

    def m_inputs_eff(self) -> torch.Tensor:
        """M_inputs as the forward uses it: the parameter itself, or its block-diagonal part when tiling is on."""
        if self.tile_size >= self.d_in:
            return self.M_inputs

        def build():
            idx = torch.arange(self.d_in, device=self.M_inputs.device) // self.tile_size
            return (self.M_inputs * (idx[:, None] == idx[None, :]).to(self.M_inputs.dtype)).contiguous()
        return self._cached("mie", (self.M_inputs,), build)

    def m_inputs_t(self) -> torch.Tensor:
        return self._cached("mit", (self.M_inputs,), lambda: self.m_inputs_eff().t().contiguous())

    def lds_params(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Poles a (S) and per-channel output weights ce, co (S,d) fitted to the even / odd lags of phi_proj.  The two
        sign branches are plus = E + O and minus = E - O (E, O the even- / odd-lag parts of the convolution): the
        decode step forms E on the bank of the token's parity and O on the other bank, and rounds the branches
        separately as the reference does (stu_utils.py:226-228, stu.py:120)."""
        def build():
            S = self.config.stu_lds_state_dim
            f = self.effective_filter()
            if f.shape[0] % 2 != 0:
                f = torch.cat([f, torch.zeros_like(f[:1])], 0)      # equally long even- and odd-lag halves
            a, ce, e1 = fit_even_lag_lds(f[0::2], S, per_channel=True)
            a2, co, e2 = fit_even_lag_lds(f[1::2], S, per_channel=True)
            if not torch.equal(a, a2):
                raise RuntimeError("pole grids of the even and odd lags differ")
            self.lds_fit_error = float(max(e1.max(), e2.max()))
            check_lds_fit(e1, f[0::2])
            check_lds_fit(e2, f[0::2])          # the odd lags against the scale of the channel's leading (even) taps
            dev = self.M_filters.device
            return a.to(dev), ce.to(dev).contiguous(), co.to(dev).contiguous()
        return self._cached("lds", (self.phi, self.M_filters), build)

    def lds_fir(self):
        """(R,d) fp32: phi_proj minus the fitted filter on the first R = stu_lds_fir_taps lags, the exact head that the
        two-branch decode step adds to the recurrence from a ring of the last R projected inputs; None when the head
        is off or does not apply (Hankel-L, exact mode, history mode)."""
        R = int(getattr(self.config, "stu_lds_fir_taps", 0) or 0)
        if R == 0 or not self.use_approx or self.use_hankel_L or self.decode_mode() != "lds":
            return None

        def build():
            a, ce, co = self.lds_params()
            f = self.effective_filter().double().cpu()
            L, d = f.shape
            fr = torch.zeros(R, d, dtype=torch.float64)
            fr[: min(R, L)] = f[: min(R, L)]                   # the reference's filter ends at lag L
            m = torch.arange(R // 2, dtype=torch.float64)
            V = a.double().cpu()[None, :] ** m[:, None]        # (R/2, S): a_j^m
            fit = torch.empty(R, d, dtype=torch.float64)
            fit[0::2] = V @ ce.double().cpu()
            fit[1::2] = V @ co.double().cpu()
            return (fr - fit).float().to(self.M_filters.device).contiguous()
        return self._cached("fir%d" % R, (self.phi, self.M_filters), build)

    def _ring_from_sequence(self, xp: torch.Tensor):
        """Ring of the last R projected inputs (position p in slot p % R, zeros before the first position), or an
        empty history slot when the exact head is off."""
        fir = self.lds_fir()
        B, T, d = xp.shape
        if fir is None:
            return xp.new_empty(B, 0, d)
        R = fir.shape[0]
        if T >= R:      # positions T-R .. T-1 to slots p % R: a rotation of the last R rows
            return torch.roll(xp[:, T - R:], shifts=(T - R) % R, dims=1).contiguous()
        ring = xp.new_zeros(B, R, d)
        ring[:, :T] = xp
        return ring

    def lds_single_params(self):
        """use_hankel_L (one branch over all lags): poles a (S) and per-channel weights ce, co (S,d) fitted to the
        even / odd lags of the effective filter; the odd lags read the other parity bank."""
        def build():
            S = self.config.stu_lds_state_dim
            f = self.effective_filter()
            a, ce, e1 = fit_even_lag_lds(f[0::2], S, per_channel=True)
            a2, co, e2 = fit_even_lag_lds(f[1::2], S, per_channel=True)
            if not torch.equal(a, a2):
                raise RuntimeError("pole grids of the even and odd lags differ")
            self.lds_fit_error = float(max(e1.max(), e2.max()))
            check_lds_fit(e1, f[0::2])
            check_lds_fit(e2, f[0::2])          # the odd lags against the scale of the channel's leading (even) taps
            dev = self.M_filters.device
            return a.to(dev), ce.to(dev).contiguous(), co.to(dev).contiguous()
        return self._cached("ldssingle", (self.phi, self.M_filters), build)

    def _single_lds_ok(self) -> bool:
        return self.use_approx and self.use_hankel_L and self.phi.shape[0] % 2 == 0

    def bank_lds_params(self):
        """Exact mode: poles a (S) and output weights ce, co (S,K) fitted to the even / odd lags of the filters."""
        def build():
            S = self.config.stu_lds_state_dim
            phi = self.phi
            a, ce, e1 = fit_even_lag_lds(phi[0::2], S)
            a2, co, e2 = fit_even_lag_lds(phi[1::2], S)       # odd lags: read from the other parity bank
            if phi.shape[0] % 2 == 0 and not torch.equal(a, a2):
                raise RuntimeError("pole grids of the even and odd lags differ")
            self.lds_fit_error = max(e1, e2)
            # the K filters are contracted together (M_phi): the error counts against the largest tap of the bank
            check_lds_fit(self.lds_fit_error, phi.detach().float().abs().max().reshape(1, 1))
            dev = phi.device
            return a.to(dev), ce.to(dev).contiguous(), co.to(dev).contiguous()
        return self._cached("banklds", (self.phi,), build)

    def exact_flat_weights_t(self):
        """(d_out, K*d_in) copies of M_phi_plus / M_phi_minus for the skinny GEMVs of a decode step."""
        def build():
            wp, wm = self.exact_flat_weights()
            return wp.t().contiguous(), (wm.t().contiguous() if wm is not None else None)
        params = (self.M_phi_plus,) + (() if self.use_hankel_L else (self.M_phi_minus,))
        return self._cached("flat_t", params, build)

    def exact_flat_weights(self):
        def build():
            Kd = self.K * self.d_in
            wp = self.M_phi_plus.reshape(Kd, self.d_out)
            wm = self.M_phi_minus.reshape(Kd, self.d_out) if not self.use_hankel_L else None
            return wp, wm
        params = (self.M_phi_plus,) + (() if self.use_hankel_L else (self.M_phi_minus,))
        return self._cached("flat", params, build)

    def _scan_prefill(self) -> bool:
        """stu_prefill_mode='scan': approx mode with both sign branches only (the recurrence is fitted to the even
        lags of the two-branch filter), 16-byte aligned rows."""
        esz = 8 if self.M_inputs.dtype == torch.bfloat16 else 4
        return (getattr(self.config, "stu_prefill_mode", "fft") == "scan" and not self.use_hankel_L
                and self.d_out % esz == 0)

    # ---- full-sequence evaluation
    def _project(self, x: torch.Tensor) -> torch.Tensor:
        B, T, d = x.shape
        if B * T <= _hip.MAX_DECODE_ROWS:
            return _hip.linear_decode(x.reshape(B * T, d), self.m_inputs_t()).reshape(B, T, self.d_out)
        x2 = x.reshape(B * T, d)
        if _hip.gemm_supported(x2, self.m_inputs_t()):
            return _hip.gemm(x2, self.m_inputs_t()).reshape(B, T, self.d_out)
        return _hip.gemm_any(x2, self.m_inputs_t()).reshape(B, T, self.d_out)

    def _convolve(self, xp: torch.Tensor) -> torch.Tensor:
        """Approx-mode convolution of the projected inputs with phi_proj (stu.py:89-98,120): the FFT form of
        the reference from FFT_MIN_T positions on, the time-domain kernel for shorter inputs and for lengths
        beyond the longest in-LDS transform."""
        T = xp.shape[1]
        n = _hip.fft_length(T) if T >= FFT_MIN_T else 0
        if n == 0:
            return _hip.stu_conv_direct(xp, self.effective_filter(), single_branch=self.use_hankel_L)
        B, _, d = xp.shape
        if self._few_long_sequences(B, T, d, xp.element_size()):
            return self._convolve_time_major(_hip.transpose(xp), n)
        return _hip.stu_conv_fft(xp, self.filter_spectrum(n), single_branch=self.use_hankel_L)

    @staticmethod
    def _few_long_sequences(B: int, T: int, d: int, esz: int) -> bool:
        """A few long sequences: the channel-contiguous FFT kernel, which takes a workgroup's 16 bytes of channels one
        after the other, would leave compute units idle, and the one-column kernel reads a (B, L, d) tensor two bytes
        at a time.  Time-major slabs let that kernel's loads and stores coalesce (measured at L=4096, d=2048, one
        row: 100 us + 8 us per transpose against 137 us), with identical results."""
        return T >= FFT_MIN_T and _hip.fft_length(T) >= 8192 and (d // (16 // esz)) * B < 512

    def _convolve_time_major(self, xt: torch.Tensor, n: int) -> torch.Tensor:
        """xt (B, d, T): the projected inputs as time-major slabs -> y (B, T, d)."""
        yt = torch.empty_like(xt)
        _hip.stu_conv_fft_strided(xt.transpose(1, 2), self.filter_spectrum(n), yt.transpose(1, 2),
                                  single_branch=self.use_hankel_L)
        return _hip.transpose(yt)

    def _project_time_major(self, x: torch.Tensor) -> Optional[torch.Tensor]:
        """(x @ M_inputs) as time-major slabs (B, d_out, T), formed by the prompt GEMM with its operands swapped
        (M_inputs^T as the rows, the sequence as the 'weights'), or None where that kernel does not take the shape."""
        B, T, d = x.shape
        w = self.m_inputs_t()
        if not all(_hip.gemm_supported(w, x[b]) for b in range(B)) or T % 4 != 0:
            return None
        xt = torch.empty(B, w.shape[0], T, dtype=x.dtype, device=x.device)
        for b in range(B):
            _hip.gemm(w, x[b], out=xt[b])
        return xt

    def _exact_sequence(self, x: torch.Tensor) -> torch.Tensor:
        """use_approx=False: U+-[b,t,k,i] for the whole filter bank (one forward transform per channel, one
        inverse per filter), then the (K*d_in, d_out) contractions on the matrix cores with the reference's
        rounding points, T(T(U+ M+) + T(U- M-)) (stu.py:107-120).  The FFT form writes U time-major, (B, K*d, T),
        which fstu_gemm_bf16_ta consumes as it lies; x is never expanded K-fold."""
        B, T, d = x.shape
        wp, wm = self.exact_flat_weights()
        n = _hip.fft_length(T) if T >= FFT_MIN_T else 0
        if n == 0:
            Up = torch.empty(B, T, self.K, d, dtype=x.dtype, device=x.device)
            Um = None if self.use_hankel_L else torch.empty_like(Up)
            _hip.stu_conv_bank(x, self.phi, Up, Um)
            wpt, wmt = self.exact_flat_weights_t()
            y = _hip.linear(Up.reshape(B * T, self.K * d), wpt)
            if Um is not None:
                y = y + _hip.linear(Um.reshape(B * T, self.K * d), wmt)
            return y.reshape(B, T, self.d_out)
        # Slabs of (K*d, Tp) per batch row with Tp = T rounded up to the contraction's 128-position tiles; the filter
        # bank writes positions below T, the contraction's rows beyond T are cut off again (each output row depends
        # on its own column of the slab only, so what the padding holds never reaches a kept row).
        Tp = (T + 127) // 128 * 128
        Kd = self.K * d
        Up = torch.empty(B, self.K, d, Tp, dtype=x.dtype, device=x.device)
        Um = None if self.use_hankel_L else torch.empty_like(Up)
        xt = x.transpose(1, 2).contiguous().transpose(1, 2)            # time-major copy: coalesced column loads
        _hip.stu_conv_bank_fft(xt, self.filter_spectrum(n), Up[..., :T].permute(0, 3, 1, 2),
                               None if Um is None else Um[..., :T].permute(0, 3, 1, 2))
        if x.dtype == torch.bfloat16 and Kd % 64 == 0 and self.d_out % 4 == 0:
            wpt, wmt = self.exact_flat_weights_t()
            y = _hip.gemm_ta(Up.view(B, Kd, Tp), wpt)
            if Um is not None:
                _hip.gemm_ta(Um.view(B, Kd, Tp), wmt, residual=y, out=y)
            return y if Tp == T else y[:, :T].contiguous()
        # fp32 (the parity path) and widths the matrix-core kernel does not take: the general kernel per batch row on
        # the (K*d, T) slab as a strided operand
        y = torch.empty(B, T, self.d_out, dtype=x.dtype, device=x.device)
        for b in range(B):
            _hip.gemm_any(Up[b].reshape(Kd, Tp)[:, :T].t(), wp.t(), out=y[b])
            if Um is not None:
                y[b] += _hip.gemm_any(Um[b].reshape(Kd, Tp)[:, :T].t(), wm.t())
        return y

    def forward_differentiable(self, x: torch.Tensor) -> torch.Tensor:
        """Training-side forward of the approx-mode STU (stu.py:81-98,120) under autograd: the two projections are
        library GEMMs, the convolution between them is the HIP kernel with its own backward
        (flash_stu.utils.stu_utils.convolve), so gradients reach x, M_inputs and M_filters.  No decode state."""
        from ..utils.stu_utils import convolve, nearest_power_of_two
        if not self.use_approx:
            raise NotImplementedError("forward_differentiable covers use_approx=True")
        if self.tile_size < self.d_in:
            raise NotImplementedError("forward_differentiable does not cover d_in_tile / d_out_tile")
        x_proj = x @ self.M_inputs
        phi_proj = self.phi @ self.M_filters
        n = nearest_power_of_two(2 * self.phi.shape[0] - 1, round_up=True)
        plus, minus = convolve(x_proj, phi_proj, n, use_approx=True, return_both=not self.use_hankel_L)
        return plus if self.use_hankel_L else plus + minus

    @torch.no_grad()
    def forward(self, x: torch.Tensor, past_state=None, use_cache: bool = False):
        """x (B,T,d).  Without past_state the whole sequence is convolved from
        position 0 (the reference's forward).  With past_state, T must be 1 and
        the call is one decode step.  Returns y, or (y, state) if use_cache."""
        x = x.contiguous()
        B, T, d = x.shape
        if past_state is None:
            if T > self.phi.shape[0]:
                raise ValueError(f"sequence length {T} exceeds the filter length {self.phi.shape[0]}")
            if self.use_approx and self._scan_prefill():
                # the distilled recurrence over the whole prompt: outputs and the decode state in one launch
                xp = self._project(x)
                a, ce, _ = self.lds_params()
                y, state = _hip.stu_scan_lds(xp, a, ce)
                if not use_cache:
                    return y
                if self.decode_mode() == "lds":
                    return y, (self._ring_from_sequence(xp), state, torch.full((B,), T, dtype=torch.int64))
                return y, self._state_from_sequence(xp)
            if self.use_approx:
                xt = None
                if not use_cache and self._few_long_sequences(B, T, self.d_out, x.element_size()):
                    xt = self._project_time_major(x)       # no transpose in front of the time-major convolution
                if xt is not None:
                    return self._convolve_time_major(xt, _hip.fft_length(T))
                xp = self._project(x)
                y = self._convolve(xp)
                hist_src = xp
            else:
                y = self._exact_sequence(x)
                hist_src = x
            if not use_cache:
                return y
            return y, self._state_from_sequence(hist_src)
        if T != 1:
            raise ValueError("a decode call with past_state takes exactly one new position")
        y, state = self._step(x.reshape(B, d), past_state)
        y = y.reshape(B, 1, self.d_out)
        return (y, state) if use_cache else y

    # ---- decode state
    def _state_from_sequence(self, src: torch.Tensor):
        B, T, d = src.shape
        pos = torch.full((B,), T, dtype=torch.int64)
        if self.decode_mode() == "lds" and (self.use_approx or self._exact_lds_ok()):
            a = (self.lds_single_params()[0] if self._single_lds_ok() else
                 self.lds_params()[0] if self.use_approx else self.bank_lds_params()[0])
            # the exact head's ring of the last projected inputs is written by the same launch on its way through them
            fir = self.lds_fir() if self.use_approx else None
            if fir is None:
                ring = None
            elif T >= fir.shape[0]:
                ring = src.new_empty(B, fir.shape[0], d)          # every slot is written
            else:
                ring = src.new_zeros(B, fir.shape[0], d)          # zeros before the first position
            state = _hip.stu_lds_state_from_hist(src.contiguous(), a, T - 1, ring=ring)
            return (ring if ring is not None else src.new_empty(B, 0, d), state, pos)
        cap = max(self.config.seq_len, T)
        hist = src.new_zeros(B, cap, d)
        hist[:, :T] = src
        return (hist, torch.empty(B, 0, dtype=torch.float32, device=src.device), pos)

    def _step(self, x: torch.Tensor, past_state):
        hist, state, pos_t = past_state
        pos = int(pos_t[0])
        B, d = x.shape
        if self.use_approx and state.numel() > 0:
            xp = _hip.linear_decode(x, self.m_inputs_t())
            if self.use_hankel_L:
                a, ce, co = self.lds_single_params()
                y = _hip.stu_step_lds(state, xp, a, ce, pos, co=co)
            else:
                a, ce, co = self.lds_params()
                fir = self.lds_fir()
                if fir is not None and hist.shape[1] == fir.shape[0]:
                    y = _hip.stu_step_lds(state, xp, a, ce, pos, co=co, pair=True, ring=hist, fir=fir)
                else:
                    y = _hip.stu_step_lds(state, xp, a, ce, pos, co=co, pair=True)
            return y, (hist, state, pos_t + 1)
        if not self.use_approx and state.numel() > 0:
            # exact mode on the recurrence state: U+- for all K filters, then the two contractions as skinny GEMVs
            a, ce, co = self.bank_lds_params()
            up, um = _hip.stu_bank_step_lds(state, x, a, ce, co, pos)
            wpt, wmt = self.exact_flat_weights_t()
            if self.use_hankel_L:
                y = _hip.linear(up.reshape(B, -1), wpt)
            else:
                y = _hip.linear(up.reshape(B, -1), wpt) + _hip.linear(um.reshape(B, -1), wmt)
            return y, (hist, state, pos_t + 1)
        if pos >= hist.shape[1]:
            hist = torch.cat([hist, torch.zeros_like(hist)], dim=1)
        if pos >= self.phi.shape[0]:
            raise ValueError(f"position {pos} is past the filter length {self.phi.shape[0]}")
        if self.use_approx:
            _hip.linear_decode(x, self.m_inputs_t(), hist[:, pos, :])
            nsplit = _hist_nsplit(pos + 1)
            eo = _hip.stu_step_hist(hist, self.effective_filter(), pos, nsplit)
            y = torch.zeros(B, d, dtype=x.dtype, device=x.device)
            _hip.add_rmsnorm(y, eo, None, 0.0, delta_mode=2, nslices=nsplit, single_branch=self.use_hankel_L,
                             want_norm=False)
            return y, (hist, state, pos_t + 1)
        # exact mode: re-evaluate the bank over the stored inputs and keep the newest row
        hist[:, pos, :] = x
        y = self._exact_sequence(hist[:, : pos + 1].contiguous())[:, -1]
        return y, (hist, state, pos_t + 1)


def _hist_nsplit(nlags: int) -> int:
    """Lag ranges per (batch) for the history kernel: enough workgroups to pull
    bandwidth without making the partial-sum traffic comparable to the history."""
    return max(1, min(16, nlags // 64))
