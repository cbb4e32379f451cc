"""Model registry: config.json -> the family that serves it.

A family registers a name (the value of config.json's "architecture", or an entry of HF's "architectures" / "model_type") and a loader
``load(path, dtype, device, **engine_args)`` returning an object with ``generate(prompts, max_new_tokens, **sampling)``.  Families that
run ragged steps also return ``run_step`` / ``release`` (scheduler.ServingEngine), which the trace replayer drives."""
import json
import os
from typing import Callable, Dict

import torch

_FAMILIES: Dict[str, Callable] = {}


def register(*names: str):
    def deco(fn):
        for n in names:
            _FAMILIES[n.lower()] = fn
        return fn
    return deco


def architecture_of(config: dict) -> str:
    if "architecture" in config:
        return str(config["architecture"])
    for a in config.get("architectures") or []:
        if a.lower() in _FAMILIES:
            return a
    return str(config.get("model_type", ""))


def families():
    return sorted(_FAMILIES)


def load_engine(path: str, dtype: torch.dtype = torch.bfloat16, device="cuda:0", **engine_args):
    """Open the checkpoint folder `path` with the family its config.json names."""
    cfg = json.load(open(os.path.join(path, "config.json")))
    arch = architecture_of(cfg)
    fn = _FAMILIES.get(arch.lower())
    if fn is None:
        raise NotImplementedError(f"{path}: architecture {arch!r} is not registered (known: {', '.join(families())})")
    return fn(path, dtype, device, **engine_args)


@register("Nufalorn", "Pokepel", "Nepudra", "Nudorax")
def _load_hybrid(path, dtype, device, *, max_tokens: int = 8192, max_seqs: int = 4, max_step_tokens: int = 2048, page: int = 64):
    from .hybrid import load_hybrid_checkpoint
    from .scheduler import ServingEngine
    return ServingEngine(load_hybrid_checkpoint(path, dtype, device, page), max_tokens=max_tokens, max_seqs=max_seqs,
                         max_step_tokens=max_step_tokens)


class _PagedDecoderRunner:
    """generate() over model.DecoderEngine for the Qwen2 / Llama family: one static batch, block tables laid out back to back."""

    def __init__(self, cfg, weights, dtype, device, max_tokens, max_seqs, page):
        from .model import DecoderEngine, weights_to
        self.page = page
        per_seq = max(1, max_tokens // max(1, max_seqs))
        self.blocks_per_seq = (per_seq + page - 1) // page
        self.engine = DecoderEngine(cfg, weights_to(weights, device), kv_int8=False, page=page, num_blocks=self.blocks_per_seq * max_seqs,
                                    max_batch=max_seqs, max_seq_len=self.blocks_per_seq * page, device=device, dtype=dtype)

    def generate(self, prompts, max_new_tokens, **sampling):
        bt = torch.arange(len(prompts) * self.blocks_per_seq, dtype=torch.int32).reshape(len(prompts), self.blocks_per_seq)
        if sampling and sampling.get("top_k", 1) != 1:
            return self.engine.generate_sampled(prompts, bt, max_new_tokens, **sampling)
        return self.engine.generate(prompts, bt, max_new_tokens)


@register("Qwen2ForCausalLM", "LlamaForCausalLM", "qwen2", "llama")
def _load_paged_decoder(path, dtype, device, *, max_tokens: int = 8192, max_seqs: int = 4, page: int = 16, quantization=None, **_):
    from .loader import load_hf_checkpoint
    if dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("the Qwen2 / Llama decode path runs in float16 or bfloat16")
    cfg, weights = load_hf_checkpoint(path, quantization=quantization, dtype=dtype)
    return _PagedDecoderRunner(cfg, weights, dtype, device, max_tokens, max_seqs, page)
