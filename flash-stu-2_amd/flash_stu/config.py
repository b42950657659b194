"""FlashSTUConfig: the reference's configuration surface
(flash_stu/config.py:71-132) without a dependency on transformers, plus the
few fields that steer the MI355X decode path."""
from __future__ import annotations

import copy
import json
import os
from typing import Any, Dict, Optional, Tuple, Union

import torch

RMS_NORM_EPS = 1.1920929e-07   # what torch.nn.RMSNorm(eps=None) uses


class FlashSTUConfig:
    model_type = "FlashSTU"

    def __init__(
        self,
        bsz: int = 1,
        n_embd: int = 1536,
        n_heads: int = 8,
        n_layers: int = 26,
        seq_len: int = 8192,
        window_size: Union[int, Tuple[int, int]] = 1024,
        vocab_size: int = 200064,
        mlp_scale: int = 12,
        bias: bool = False,
        dropout: float = 0.0,
        num_eigh: int = 24,
        use_hankel_L: bool = False,
        use_flash_fft: bool = True,
        use_approx: bool = True,
        use_attn: bool = True,
        use_cache: bool = True,
        use_gradient_checkpointing: bool = False,
        softcap: float = 50.0,
        torch_dtype: Union[torch.dtype, str, None] = torch.bfloat16,
        tie_word_embeddings: bool = True,
        stu_enable_mlp_sandwich: bool = False,
        stu_mlp_hidden_size: Optional[int] = None,
        filter_path: Optional[str] = None,
        d_in_tile: Optional[int] = None,
        d_out_tile: Optional[int] = None,
        # --- decode path of this implementation ---
        rms_norm_eps: float = RMS_NORM_EPS,
        stu_decode_mode: str = "auto",       # "history" (exact), "lds" (distilled recurrence), "auto": lds for bf16
        stu_lds_state_dim: int = 64,
        stu_lds_fir_taps: int = 64,          # exact head of the distilled filter: first lags taken from phi_proj itself (0: off)
        stu_prefill_mode: str = "fft",       # "fft": the reference's convolution; "scan": the distilled recurrence over the prompt
        **kwargs: Any,
    ):
        self.bsz = bsz
        self.n_embd = n_embd
        self.n_heads = n_heads
        self.n_layers = n_layers
        self.seq_len = seq_len
        self.window_size = window_size
        self.vocab_size = vocab_size
        self.hidden_size = n_embd
        self.intermediate_size = n_embd * mlp_scale
        self.hidden_act = "swish"
        self.bias = bias
        self.dropout = dropout
        self.num_eigh = num_eigh
        self.use_hankel_L = use_hankel_L
        self.use_flash_fft = use_flash_fft
        self.use_approx = use_approx
        self.use_attn = use_attn
        self.use_cache = use_cache
        self.use_gradient_checkpointing = use_gradient_checkpointing
        self.softcap = softcap
        self.stu_enable_mlp_sandwich = stu_enable_mlp_sandwich
        self.stu_mlp_hidden_size = stu_mlp_hidden_size
        self.filter_path = filter_path
        self.d_in_tile = d_in_tile
        self.d_out_tile = d_out_tile
        if torch_dtype is None:
            self.torch_dtype = torch.float32
        elif isinstance(torch_dtype, str):
            self.torch_dtype = getattr(torch, torch_dtype.replace("torch.", ""))
        else:
            self.torch_dtype = torch_dtype
        self.mlp_scale = mlp_scale
        self.tie_word_embeddings = tie_word_embeddings
        self.rms_norm_eps = rms_norm_eps
        if stu_decode_mode not in ("auto", "history", "lds"):
            raise ValueError(f"stu_decode_mode must be auto|history|lds, got {stu_decode_mode!r}")
        self.stu_decode_mode = stu_decode_mode
        self.stu_lds_state_dim = stu_lds_state_dim
        if stu_lds_fir_taps and (stu_lds_fir_taps < 8 or stu_lds_fir_taps > 1024 or stu_lds_fir_taps & (stu_lds_fir_taps - 1)):
            raise ValueError(f"stu_lds_fir_taps must be 0 or a power of two in 8..1024, got {stu_lds_fir_taps}")
        self.stu_lds_fir_taps = int(stu_lds_fir_taps)
        if stu_prefill_mode not in ("fft", "scan"):
            raise ValueError(f"stu_prefill_mode must be fft|scan, got {stu_prefill_mode!r}")
        self.stu_prefill_mode = stu_prefill_mode
        self.use_return_dict = kwargs.pop("return_dict", True)
        self.output_hidden_states = kwargs.pop("output_hidden_states", False)
        for k, v in kwargs.items():          # unknown keys are kept, as PretrainedConfig does
            setattr(self, k, v)

    # -- window as the left extent the kernels use
    @property
    def window_left(self) -> int:
        w = self.window_size
        return int(w[0]) if isinstance(w, (tuple, list)) else int(w)

    def resolved_stu_decode_mode(self) -> str:
        if self.stu_decode_mode != "auto":
            return self.stu_decode_mode
        bf16 = self.torch_dtype == torch.bfloat16
        if not self.use_approx:
            # exact mode decodes on the recurrence state of the raw inputs when the filters can be split into equal
            # even / odd lag halves and fit the bank kernel; otherwise it re-evaluates the bank over the history
            return "lds" if (bf16 and self.seq_len % 2 == 0 and self.num_eigh <= 32) else "history"
        if self.use_hankel_L:
            # one branch over all lags: even lags from the bank of the token's parity, odd lags from the other bank
            return "lds" if (bf16 and self.seq_len % 2 == 0) else "history"
        return "lds" if bf16 else "history"

    # -- serialisation (config.json, HF style)
    def to_dict(self) -> Dict[str, Any]:
        out = copy.deepcopy({k: v for k, v in self.__dict__.items() if not k.startswith("_")})
        out["torch_dtype"] = str(self.torch_dtype).replace("torch.", "")
        out["model_type"] = self.model_type
        if isinstance(out.get("window_size"), tuple):
            out["window_size"] = list(out["window_size"])
        out["return_dict"] = out.pop("use_return_dict")
        return out

    def to_json_string(self) -> str:
        return json.dumps(self.to_dict(), indent=2, sort_keys=True) + "\n"

    @classmethod
    def from_dict(cls, d: Dict[str, Any], **kw) -> "FlashSTUConfig":
        d = dict(d)
        d.update(kw)
        for drop in ("model_type", "hidden_size", "intermediate_size", "hidden_act", "transformers_version",
                     "architectures", "dtype"):
            d.pop(drop, None)
        if isinstance(d.get("window_size"), list):
            d["window_size"] = tuple(d["window_size"])
        return cls(**d)

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            f.write(self.to_json_string())

    @classmethod
    def from_pretrained(cls, path: str, **kw) -> "FlashSTUConfig":
        p = os.path.join(path, "config.json") if os.path.isdir(path) else path
        with open(p) as f:
            return cls.from_dict(json.load(f), **kw)

    def __repr__(self) -> str:
        return f"FlashSTUConfig {self.to_json_string()}"
