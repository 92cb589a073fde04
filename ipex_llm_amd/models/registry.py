"""Native architectures: checkpoints in their own layout (no HF model class).

Such a folder's ``config.json`` names its design under ``"architecture"``;
the table below maps that name to the module that reads the configuration
and the weights (``load(path, dtype, device)``) into a model the engines
drive directly.  ``AutoModelForCausalLM.from_pretrained``, the command line
and the trace replayer consult it before anything HF-shaped.
"""
from __future__ import annotations

import importlib
import json
import os
from typing import List, Optional

import torch

NATIVE_ARCHITECTURES = {
    "Zamelix": "ipex_llm_amd.models.zamelix",
    "Masezen": "ipex_llm_amd.models.masezen",
    "Vogolix": "ipex_llm_amd.models.vogolix",
    "Zoguzen": "ipex_llm_amd.models.zoguzen",
}


def native_architecture(path) -> Optional[str]:
    """the registered architecture a checkpoint folder names, else None"""
    cfg = os.path.join(str(path), "config.json")
    if not os.path.isfile(cfg):
        return None
    try:
        with open(cfg) as f:
            arch = json.load(f).get("architecture")
    except (OSError, ValueError):
        return None
    return arch if isinstance(arch, str) and arch in NATIVE_ARCHITECTURES else None


def load_native(path, dtype=torch.bfloat16, device="cuda"):
    arch = native_architecture(path)
    if arch is None:
        raise ValueError(f"{path}: no registered native architecture in config.json")
    return importlib.import_module(NATIVE_ARCHITECTURES[arch]).load(str(path), dtype=dtype, device=device)


class NativeCheckpointLM:
    """``generate()`` facade over a natively loaded model: token ids in,
    token ids out, through the continuous-batching engine (its scheduler,
    cache and sampler)."""

    def __init__(self, path, dtype=torch.bfloat16, device="cuda"):
        self.path, self.dtype = str(path), dtype
        self.model = load_native(path, dtype, device)
        self.config = getattr(self.model, "config", None)
        self._engine = None

    @property
    def device(self):
        return self.model.device

    def to(self, device):
        if torch.device(device) != self.model.device:
            self.model = self.model.to(device)
            for L in self.model.layers:
                if hasattr(L.mixer, "table"):
                    L.mixer.table = None
            self._engine = None
        return self

    def eval(self):
        return self

    def engine(self, max_batch: int = 8, max_model_len: int = 4096, **kw):
        from ..serving.engine import LLMEngine
        if self._engine is None or self._engine.max_model_len < max_model_len:
            self._engine = LLMEngine(self.model, max_batch=max_batch, max_model_len=max_model_len,
                                     max_prefill_tokens=kw.pop("max_prefill_tokens", 2048), **kw)
        return self._engine

    @torch.no_grad()
    def generate(self, input_ids, max_new_tokens: int = 32, do_sample: bool = False, temperature: float = 1.0,
                 top_k: int = 0, top_p: float = 1.0, repetition_penalty: float = 1.0, eos_token_id=None,
                 pad_token_id: int = 0, **_):
        from ..serving.engine import SamplingParams
        rows: List[List[int]] = input_ids.tolist() if isinstance(input_ids, torch.Tensor) else [list(r) for r in input_ids]
        eng = self.engine(max_batch=max(8, len(rows)), max_model_len=max(len(r) for r in rows) + max_new_tokens + 1)
        eos = [eos_token_id] if isinstance(eos_token_id, int) else list(eos_token_id or [])
        gen = eng.generate(rows, SamplingParams(max_new_tokens=max_new_tokens, do_sample=do_sample,
                                                temperature=temperature, top_k=top_k, top_p=top_p,
                                                repetition_penalty=repetition_penalty, stop_token_ids=eos))
        if not isinstance(input_ids, torch.Tensor):
            return [r + g for r, g in zip(rows, gen)]
        width = max(len(r) + len(g) for r, g in zip(rows, gen))
        out = torch.full((len(rows), width), pad_token_id, dtype=input_ids.dtype)
        for i, (r, g) in enumerate(zip(rows, gen)):
            out[i, :len(r) + len(g)] = torch.tensor(r + g, dtype=input_ids.dtype)
        return out.to(input_ids.device)
