"""Text-only language models on the hybrid engine (`engine_hybrid.HybridEngine`): the part of the plugin that does not depend on
the design.  A design gives `config_from_dict` (config.json -> HybridCfg) and `pack_weights` (checkpoint tensors -> the engine's
fused layout); forward, sampling and the next-step feedback are one native call per step.  There is no audio side: generated ids
are the output."""
import json
import os
from typing import Dict, List, Optional

import torch

from ..engine_hybrid import HybridCfg, HybridEngine
from ..sampling import SamplingConfig
from .base import BaseLM, PreprocessOutput


class HybridLM(BaseLM):
    """`preprocess` takes token ids (a list / tensor under `token_ids`, or a prompt of whitespace-separated ids), the request's
    output is its generated ids (`lm_output_tokens`)."""

    stop_token_ids: List[int] = []
    default_name = "hybrid-lm"

    @staticmethod
    def config_from_dict(d: dict) -> HybridCfg:
        raise NotImplementedError

    @staticmethod
    def pack_weights(S: Dict[str, torch.Tensor], cfg: HybridCfg) -> Dict:
        raise NotImplementedError

    def __init__(self, model_name, weights: Dict[str, torch.Tensor], config: HybridCfg, device="cuda:0", dtype=torch.bfloat16,
                 audio_decoder_device=None, max_batch_size=8, page_size=128, max_num_pages=256, max_seq_len=4096,
                 max_prefill_tokens=1024, max_logit_rows=None, state_slots=None, sampling: Optional[SamplingConfig] = None,
                 max_tokens=1024, stop_token_ids=None, **_ignored):
        super().__init__(model_name, device, dtype, False, audio_decoder_device)
        self.config = config
        self.default_sampling_config = sampling or SamplingConfig(top_k=None, top_p=None, min_p=None, temperature=1.0, max_tokens=max_tokens,
                                                                  repetition_penalty=None, repetition_window=None, cfg_scale=None, greedy=True)
        self._max_tokens = max_tokens
        if stop_token_ids is not None:
            self.stop_token_ids = list(stop_token_ids)
        self.engine = HybridEngine(config, self.pack_weights(weights, config), dtype=dtype, max_batch=max_batch_size, page_size=page_size,
                                   max_pages=max_num_pages, max_seq_len=max_seq_len, max_prefill_rows=max_prefill_tokens,
                                   max_out=max_logit_rows, state_slots=state_slots, device=device)

    @classmethod
    def from_checkpoint(cls, path, **kw):
        from safetensors.torch import load_file
        with open(os.path.join(path, "config.json")) as f:
            cfg = cls.config_from_dict(json.load(f))
        return cls(kw.pop("model_name", cls.default_name), load_file(os.path.join(path, "model.safetensors")), cfg, **kw)

    n_codebooks = property(lambda self: 1)
    num_attention_heads = property(lambda self: max(m.heads for m in self.config.layers))
    num_key_value_heads = property(lambda self: max([m.kv_heads for m in self.config.layers if m.kv_heads] or [0]))
    num_hidden_layers = property(lambda self: len(self.config.runs()))
    hidden_size = property(lambda self: self.config.width)
    vocab_size = property(lambda self: self.config.vocab)
    # no audio side: the windows below are never decoded (nothing is appended to lm_output_audio_tokens)
    detokenize_interval = property(lambda self: 1)
    detokenize_overlap = property(lambda self: 0)
    output_audio_length = property(lambda self: 0)
    max_tokens = property(lambda self: self.default_sampling_config.max_tokens or self._max_tokens)
    has_recurrent_state = True

    def is_stop_id(self, token_ids) -> bool:
        t = token_ids[0] if hasattr(token_ids, "__len__") else token_ids
        return int(t) in self.stop_token_ids

    def preprocess(self, prompt: str = None, audio_path: str = None, token_ids=None, **kwargs) -> PreprocessOutput:
        if token_ids is None:
            token_ids = [int(t) for t in (prompt or "").split()]
        ids = torch.as_tensor(token_ids, dtype=torch.long).view(-1, 1)
        if ids.numel() == 0:
            raise ValueError("empty prompt")
        if int(ids.min()) < 0 or int(ids.max()) >= self.vocab_size:
            raise ValueError(f"token id outside [0, {self.vocab_size})")
        return PreprocessOutput(input_tokens=ids)

    def update_requests(self, requests, out: torch.Tensor):
        """out [B,1] int64 on the host: the request-state half of sampling."""
        for i, req in enumerate(requests):
            row = out[i:i + 1].clone()
            req.input_tokens = row
            req.lm_output_tokens.append(row)
            if int(row[0, 0]) in self.stop_token_ids:
                req.done_lm_generation = True
                req.finish_reason = "stop_id_encountered"
            elif len(req.lm_output_tokens) >= self.max_tokens:
                req.done_lm_generation = True
                req.finish_reason = "max_tokens_reached"

    def postprocess(self, token_ids: torch.Tensor, **kwargs) -> torch.Tensor:
        raise NotImplementedError("this model generates token ids; there is no waveform to decode")
