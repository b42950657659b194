"""FlashSTU language model (reference: flash_stu/model.py:26-513) on the
MI355X HIP path.

The class keeps the reference's constructor, `forward`, `generate` and helper
methods.  `forward` evaluates a whole sequence (library GEMMs + the HIP
convolution / attention / norm kernels) or one decode step against the caches
it returned earlier; `generate` runs the token loop on the fused decode engine
(flash_stu/engine.py).  Inference only: every forward runs under no_grad.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _hip
from .config import FlashSTUConfig
from .layers.attention_layer import AttentionLayer
from .layers.stu_layer import STULayer
from .modules.attention import Attention
from .modules.norm import RMSNorm
from .modules.stu import STU
from .utils.numerics import nearest_power_of_two
from .utils.stu_utils import get_spectral_filters


@dataclass
class CausalLMOutputWithPast:
    """Attribute- and key-addressable output, the fields generate() and user
    code read from the reference's transformers output object."""
    loss: Optional[torch.Tensor] = None
    logits: Optional[torch.Tensor] = None
    past_key_values: Optional[Tuple] = None
    hidden_states: Optional[Tuple] = None

    def __getitem__(self, k):
        if isinstance(k, str):
            return getattr(self, k)
        return tuple(v for v in (self.loss, self.logits, self.past_key_values, self.hidden_states) if v is not None)[k]

    def get(self, k, default=None):
        v = getattr(self, k, default)
        return default if v is None else v

    def keys(self):
        return [k for k in ("loss", "logits", "past_key_values", "hidden_states") if getattr(self, k) is not None]


class FlashSTU(nn.Module):
    config_class = FlashSTUConfig
    _tied_weights_keys = ["lm_head.weight"]

    def __init__(self, config: FlashSTUConfig) -> None:
        super().__init__()
        self.config = config
        self.n_layers = config.n_layers
        self.n = nearest_power_of_two(config.seq_len * 2 - 1, round_up=True)
        self.use_approx = config.use_approx
        self.use_hankel_L = config.use_hankel_L
        phi = get_spectral_filters(config.seq_len, config.num_eigh, use_hankel_L=config.use_hankel_L,
                                   device=torch.device("cpu"), dtype=config.torch_dtype, load_from=config.filter_path)
        self.register_buffer("phi", phi, persistent=True)
        self.tok_emb = nn.Embedding(config.vocab_size, config.n_embd, dtype=config.torch_dtype)
        self.layers = nn.ModuleList()
        for idx in range(self.n_layers):
            if idx % 2 == 0 or not config.use_attn:
                self.layers.append(STULayer(config, self.phi, self.n))
            else:
                self.layers.append(AttentionLayer(config))
        self.norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.lm_head = nn.Linear(config.n_embd, config.vocab_size, bias=config.bias, dtype=config.torch_dtype)   # model.py:100-102
        self.tok_emb.weight = self.lm_head.weight
        self.std = config.n_embd ** -0.5
        self.apply(self._init_weights)
        self._engine = None

    # ------------------------------------------------------------ init
    def _init_weights(self, module):
        """model.py:428-452, including the model-level std that every SCALE_INIT
        linear shrinks for all modules visited after it."""
        if isinstance(module, nn.Linear):
            if hasattr(module, "SCALE_INIT"):
                self.std *= (2 * self.n_layers) ** -0.5
            torch.nn.init.normal_(module.weight, mean=0.0, std=self.std)
            if module.bias is not None:
                torch.nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            torch.nn.init.normal_(module.weight, mean=0.0, std=self.std)
        elif isinstance(module, STU):
            if self.use_approx:
                torch.nn.init.xavier_normal_(module.M_inputs)
                torch.nn.init.xavier_normal_(module.M_filters)
            else:
                torch.nn.init.xavier_normal_(module.M_phi_plus)
                if not self.use_hankel_L:
                    torch.nn.init.xavier_normal_(module.M_phi_minus)
        elif isinstance(module, Attention):
            torch.nn.init.xavier_normal_(module.c_attn.weight)
            torch.nn.init.xavier_normal_(module.c_proj.weight)
            for lin in (module.c_attn, module.c_proj):
                if lin.bias is not None:
                    torch.nn.init.zeros_(lin.bias)

    @torch.no_grad()
    def load_named_tensors(self, w: Dict[str, torch.Tensor]) -> None:
        """Copies a {reference state-dict name: tensor} mapping into the model."""
        sd = self.state_dict()
        for k, v in w.items():
            if k == "lm_head.weight":
                continue
            if k not in sd:
                raise KeyError(k)
            sd[k].copy_(v)
        for layer in self.layers:
            if isinstance(layer, STULayer):
                layer.stu.phi.copy_(self.phi)

    # ------------------------------------------------------------ forward
    def _embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        return _hip.embed(input_ids, self.tok_emb.weight)

    def _head(self, x: torch.Tensor) -> torch.Tensor:
        return _hip.linear(x, self.lm_head.weight, self.lm_head.bias)

    @torch.no_grad()
    def _run_layers(self, x, past_key_values, use_cache, hidden):
        cache = []
        for idx, layer in enumerate(self.layers):
            past = past_key_values[idx] if past_key_values is not None else None
            if use_cache or past is not None:
                x, present = layer(x, past_key_value=past, use_cache=True)
                cache.append(present)
            else:
                x = layer(x, past_key_value=None, use_cache=False)
            if hidden is not None:
                hidden.append(x.clone())
        return x, (tuple(cache) if use_cache else None)

    @torch.no_grad()
    def forward(self, input_ids: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None,
                past_key_values: Optional[Tuple] = None, labels: Optional[torch.LongTensor] = None,
                use_cache: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                return_dict: Optional[bool] = None, **kwargs):
        """model.py:108-205.  With past_key_values, input_ids holds the new
        positions only; several new positions are fed one at a time."""
        return_dict = return_dict if return_dict is not None else getattr(self.config, "use_return_dict", True)
        use_cache = use_cache if use_cache is not None else getattr(self.config, "use_cache", False)
        output_hidden_states = bool(output_hidden_states)
        if input_ids is None:
            raise ValueError("input_ids must be provided")
        if not input_ids.is_cuda:
            raise _hip.FlashSTUHipError("input_ids must be on the GPU: this model has no CPU path")
        hidden = [] if output_hidden_states else None
        if past_key_values is not None and input_ids.shape[1] > 1:
            outs = []
            cache = past_key_values
            for t in range(input_ids.shape[1]):
                x = self._embed(input_ids[:, t:t + 1])
                x, cache = self._run_layers(x, cache, True, None)
                outs.append(self.norm(x))
            xn = torch.cat(outs, dim=1)
            cache = cache if use_cache else None
        else:
            x = self._embed(input_ids)
            if hidden is not None:
                hidden.append(x.clone())
            x, cache = self._run_layers(x, past_key_values, use_cache, hidden)
            xn = self.norm(x)
        if kwargs.get("last_only"):        # generate() needs the newest position only (the reference computes all)
            xn = xn[:, -1:, :].contiguous()
        logits = self._head(xn)
        loss = None
        if labels is not None:
            sl = logits[..., :-1, :].contiguous()
            loss = F.cross_entropy(sl.view(-1, sl.size(-1)).float(), labels[..., 1:].contiguous().view(-1))
        hs = tuple(hidden) if hidden is not None else None
        if not return_dict:
            out = (logits,)
            if use_cache:
                out = out + (cache,)
            if output_hidden_states:
                out = out + (hs,)
            return ((loss,) + out) if loss is not None else out
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=cache, hidden_states=hs)

    # ------------------------------------------------------------ generate
    def decode_engine(self):
        from .engine import DecodeEngine
        if self._engine is None:
            self._engine = DecodeEngine(self)
        return self._engine

    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor, max_length: int = 100, temperature: float = 1.0,
                 top_k: Optional[int] = None, top_p: Optional[float] = None, do_sample: bool = True,
                 use_cache: bool = True, seed: int = 0, return_logits: bool = False, **kwargs) -> torch.LongTensor:
        """model.py:207-304: returns (B, max_length) ids, max_length counting the
        prompt.  use_cache=True runs prefill once and then one fused decode step
        per token; use_cache=False re-runs the whole sequence every step as the
        reference does.  Sampling draws come from a counter-based stream keyed
        by (seed, step, row) instead of torch's global generator."""
        B, P = input_ids.shape
        n_new = max_length - P
        if n_new <= 0:
            return input_ids
        from .engine import DecodeEngine
        # Sequences that outgrow seq_len leave the stateful paths: the filters end at lag seq_len, so the reference
        # re-runs the last seq_len tokens without a cache from there on (model.py:250-255), and so does the loop below.
        if use_cache and max_length <= self.config.seq_len and DecodeEngine.supports(self.config):
            return self.decode_engine().generate(input_ids, n_new, temperature, top_k, top_p, do_sample, seed,
                                                 return_logits=return_logits, use_graph=kwargs.get("use_graph", True))
        tokens = torch.empty(B, max_length, dtype=torch.int64, device=input_ids.device)
        tokens[:, :P] = input_ids
        all_logits = []
        if use_cache and max_length <= self.config.seq_len:
            # variants the one-call decode step does not cover (exact mode, sandwich, biases): the same token loop
            # over the layers' own decode state, one forward(use_cache=True) per token as the reference loops
            past = None
            for step in range(n_new):
                cur = P + step
                inp = tokens[:, :cur] if past is None else tokens[:, cur - 1:cur]
                out = self.forward(inp.contiguous(), past_key_values=past, use_cache=True, last_only=True)
                past = out.past_key_values
                last = out.logits[:, -1, :].contiguous()
                if return_logits:
                    all_logits.append(last)
                _hip.sample(last, tokens[:, cur], temperature, top_k, top_p, do_sample, seed, step)
            return (tokens, torch.stack(all_logits, 1)) if return_logits else tokens
        for step in range(n_new):
            cur = P + step
            lo = max(0, cur - self.config.seq_len)
            out = self.forward(tokens[:, lo:cur].contiguous(), use_cache=False)
            last = out.logits[:, -1, :].contiguous()
            if return_logits:
                all_logits.append(last)
            _hip.sample(last, tokens[:, cur], temperature, top_k, top_p, do_sample, seed, step)
        return (tokens, torch.stack(all_logits, 1)) if return_logits else tokens

    def prepare_inputs_for_generation(self, input_ids, past_key_values=None, attention_mask=None, use_cache=None,
                                      **kwargs) -> Dict[str, Any]:
        if past_key_values is not None:
            input_ids = input_ids[:, -1:]
        return {"input_ids": input_ids, "past_key_values": past_key_values, "use_cache": use_cache,
                "attention_mask": attention_mask}

    @staticmethod
    def _reorder_cache(past_key_values, beam_idx: torch.Tensor):
        """model.py:404-426: every cache entry is a tuple of batch-first tensors."""
        out = ()
        for layer_past in past_key_values:
            if layer_past is None:
                out += (None,)
            else:
                out += (tuple(t.index_select(0, beam_idx.to(t.device)) for t in layer_past),)
        return out

    # ------------------------------------------------------------ bookkeeping
    def get_num_params(self, non_embedding: bool = False) -> int:
        n = sum(p.numel() for p in self.parameters())   # tied weight counted once by parameters()
        if non_embedding:
            n -= self.tok_emb.weight.numel()
        return n

    def _get_num_params(self):
        return self.get_num_params(non_embedding=False)

    def resize_token_embeddings(self, new_num_tokens: int) -> nn.Embedding:
        old = self.config.vocab_size
        if new_num_tokens == old:
            return self.tok_emb
        dev, dt = self.lm_head.weight.device, self.config.torch_dtype
        head = nn.Linear(self.config.n_embd, new_num_tokens, bias=self.lm_head.bias is not None, dtype=dt).to(dev)
        torch.nn.init.normal_(head.weight, mean=0.0, std=self.std)
        keep = min(old, new_num_tokens)
        head.weight.data[:keep] = self.lm_head.weight.data[:keep]
        if head.bias is not None:
            torch.nn.init.zeros_(head.bias)
            head.bias.data[:keep] = self.lm_head.bias.data[:keep]
        emb = nn.Embedding(new_num_tokens, self.config.n_embd, dtype=dt).to(dev)
        self.lm_head, self.tok_emb = head, emb
        self.tok_emb.weight = self.lm_head.weight
        self.config.vocab_size = new_num_tokens
        self._engine = None
        return self.tok_emb

    def save_pretrained(self, save_directory: str, **kwargs) -> None:
        """config.json + model.safetensors with the reference's parameter names
        (tied lm_head.weight is not duplicated)."""
        from safetensors.torch import save_file
        os.makedirs(save_directory, exist_ok=True)
        self.config.save_pretrained(save_directory)
        sd = {k: v.detach().cpu().contiguous() for k, v in self.state_dict().items() if k != "lm_head.weight"}
        save_file(sd, os.path.join(save_directory, "model.safetensors"), metadata={"format": "pt"})

    @classmethod
    def from_pretrained(cls, path: str, **kwargs) -> "FlashSTU":
        """Loads a directory written by save_pretrained here or by the reference (config.json +
        model.safetensors, or sharded model-*.safetensors with model.safetensors.index.json; model.py:338-366),
        or a single training checkpoint file model_<step>.safetensors (training/distributed.py:140-148) together
        with config=...  Only safetensors are read: nothing in a checkpoint is ever executed."""
        from safetensors.torch import load_file
        import json
        if os.path.isfile(path):
            config = kwargs.pop("config", None)
            if config is None:
                cj = os.path.join(os.path.dirname(path), "config.json")
                if not os.path.exists(cj):
                    raise ValueError("a bare .safetensors checkpoint needs config=FlashSTUConfig(...) or a config.json beside it")
                config = FlashSTUConfig.from_pretrained(cj)
            sd = load_file(path)
        else:
            config = kwargs.pop("config", None) or FlashSTUConfig.from_pretrained(path)
            index = os.path.join(path, "model.safetensors.index.json")
            if os.path.exists(index):
                with open(index) as f:
                    shards = sorted(set(json.load(f)["weight_map"].values()))
                sd = {}
                for sh in shards:
                    sd.update(load_file(os.path.join(path, sh)))
            else:
                sd = load_file(os.path.join(path, "model.safetensors"))
        model = cls(config)
        sd = {(k[len("module."):] if k.startswith("module.") else k): v for k, v in sd.items()}   # DDP-wrapped saves
        sd = {(k[len("_orig_mod."):] if k.startswith("_orig_mod.") else k): v for k, v in sd.items()}  # compiled saves
        if "lm_head.weight" in sd and "tok_emb.weight" not in sd:
            sd["tok_emb.weight"] = sd.pop("lm_head.weight")
        sd.pop("lm_head.weight", None)
        missing, unexpected = model.load_state_dict(sd, strict=False)
        missing = [m for m in missing if m != "lm_head.weight"]
        if missing or unexpected:
            raise RuntimeError(f"checkpoint mismatch: missing {missing}, unexpected {unexpected}")
        for layer in model.layers:
            if isinstance(layer, STULayer):
                layer.stu.phi.copy_(model.phi)
        return model
