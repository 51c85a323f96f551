"""Generation loop of the reference (src/generation.rs) over the HIP model step.

The reference copies the logits to the host after every token, samples there with thread_rng and
uploads the token (src/generation.rs:114-124).  Here the draw happens on the device
(bdh_sample_top_k): the uniform variates come from a torch generator on the GPU, the sampled token is
fed back without leaving HBM, and the only host transfers are the ones the caller asks for (streaming
callback or the final token list).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch

from .model.bdh import BDH
from .model.state import ModelState
from .tokenizer import Tokenizer


@dataclass(frozen=True)
class ContextStrategy:
    """src/generation.rs:12-16: Infinite, or Sliding { window }."""

    window: Optional[int] = None  # None = Infinite

    @classmethod
    def infinite(cls) -> "ContextStrategy":
        return cls(None)

    @classmethod
    def sliding(cls, window: int) -> "ContextStrategy":
        return cls(int(window))


@dataclass
class GenerationSettings:
    """src/generation.rs:18-24."""

    max_new_tokens: Optional[int] = None
    temperature: float = 1.0
    top_k: Optional[int] = None
    strategy: ContextStrategy = ContextStrategy()


@dataclass
class GenerationConfig:
    """src/config/core.rs:20-30."""

    prompt: str = ""
    max_tokens: Optional[int] = None
    temperature: float = 1.0
    top_k: Optional[int] = None
    context_strategy: ContextStrategy = ContextStrategy()


def resolve_context_strategy(strategy: ContextStrategy, default_window: int) -> ContextStrategy:
    """src/generation.rs:243-259: a sliding window of 0 means the training block size."""
    if strategy.window is None:
        return strategy
    return ContextStrategy(max(default_window, 1) if strategy.window == 0 else strategy.window)


def normalize_max_tokens(max_tokens: Optional[int]) -> Optional[int]:
    """src/generation.rs:236-241: negative means unbounded."""
    return max_tokens if max_tokens is not None and max_tokens >= 0 else None


def sample_from_logits(model: BDH, last_logits: torch.Tensor, temperature: float, top_k: Optional[int],
                       uniforms: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sample_from_logits_values after the temperature division (src/generation.rs:26-72,117), on the
    device.  last_logits [B,V] f32 (rows may be strided), uniforms [B] f32 in [0,1) -> tokens [B] int64."""
    assert last_logits.dim() == 2 and last_logits.stride(1) == 1 and last_logits.dtype == torch.float32
    B, V = last_logits.shape
    uniforms = uniforms.to(last_logits.device, torch.float32).contiguous()
    assert uniforms.numel() == B
    if out is None:
        out = torch.empty((B,), device=last_logits.device, dtype=torch.int64)
    ctx = model.ctx
    ctx.check(ctx.lib.bdh_sample_top_k(ctx.handle, B, V, last_logits.data_ptr(), last_logits.stride(0) if B > 1 else V,
                                       float(temperature), int(top_k) if top_k else 0, uniforms.data_ptr(),
                                       out.data_ptr()))
    return out


def prefill_state(model: BDH, prompt_tokens) -> Tuple[ModelState, torch.Tensor]:
    """src/generation.rs:74-105: runs the prompt through forward_with_state on a fresh state and
    returns the state and the logits of the last prompt token [V]."""
    prompt = torch.as_tensor(prompt_tokens, dtype=torch.int64).reshape(1, -1)
    if prompt.shape[1] == 0:
        raise ValueError("prompt must contain at least one token")
    state = model.init_state()
    logits = model.forward_with_state(prompt, state)
    if logits.shape[1] != prompt.shape[1]:
        raise RuntimeError(f"prefill produced mismatched length: expected {prompt.shape[1]}, got {logits.shape[1]}")
    return state, logits[0, -1]


def uniform_variates(n: int, device, generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """n uniform variates in [0, 1) as an [n] tensor on `device`, drawn on the generator's own device (a CPU
    generator serves a GPU model)."""
    if generator is not None and generator.device.type != torch.device(device).type:
        return torch.rand((n,), device=generator.device, generator=generator).to(device)
    return torch.rand((n,), device=device, generator=generator)


class VariateStream:
    """The uniform variates of one generation run, drawn from `generator` a block at a time so that no host work
    is done per token.  Every consumer draws blocks of the same size: two runs from equal seeds see the same
    sequence whichever entry point they go through."""

    BLOCK = 256

    def __init__(self, device, generator: Optional[torch.Generator] = None):
        self.device, self.generator = device, generator
        self._buf, self._at = None, 0

    def next(self) -> torch.Tensor:
        if self._buf is None or self._at == self.BLOCK:
            self._buf, self._at = uniform_variates(self.BLOCK, self.device, self.generator), 0
        self._at += 1
        return self._buf[self._at - 1:self._at]


def sample_next_token(model: BDH, state: ModelState, last_logits: torch.Tensor, temperature: float,
                      top_k: Optional[int], generator: Optional[torch.Generator] = None,
                      variates: Optional[VariateStream] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """src/generation.rs:107-128: draws from last_logits [V], feeds the token and returns
    (token [1] int64 on the device, logits of the new token [V]).  The variate comes from `variates` when a
    run keeps a stream, else from a draw of its own."""
    u = variates.next() if variates is not None else uniform_variates(1, last_logits.device, generator)
    nxt = sample_from_logits(model, last_logits.reshape(1, -1), temperature, top_k, u)
    logits = model.forward_with_state(nxt.reshape(1, 1), state)
    return nxt, logits[0, -1]


def generate_tokens(model: BDH, prompt_tokens: List[int], settings: GenerationSettings,
                    on_token: Optional[Callable[[int], None]] = None,
                    generator: Optional[torch.Generator] = None) -> List[int]:
    """src/generation.rs:158-203.  Without a callback the tokens stay on the device until the end;
    with one, each token is copied to the host as it is produced (streaming)."""
    if settings.max_new_tokens is None and on_token is None:
        raise ValueError("an unbounded generation needs an on_token callback that eventually raises StopIteration")
    full = list(int(t) for t in prompt_tokens)
    state, last_logits = prefill_state(model, full)
    window = settings.strategy.window
    if window and state.position > window:
        state.trim(window)
    produced: List[torch.Tensor] = []
    generated = 0
    variates = VariateStream(last_logits.device, generator)
    try:
        while settings.max_new_tokens is None or generated < settings.max_new_tokens:
            nxt, last_logits = sample_next_token(model, state, last_logits, settings.temperature, settings.top_k,
                                                 generator, variates)
            generated += 1
            if on_token is not None:
                tok = int(nxt[0])
                full.append(tok)
                on_token(tok)
            else:
                produced.append(nxt)
            if window and state.position > window:
                state.trim(window)
    except StopIteration:
        pass
    if produced:
        full.extend(int(t) for t in torch.cat(produced).cpu())
    return full


def generate_text(model: BDH, tokenizer: Tokenizer, block_size: int, generation: GenerationConfig,
                  generator: Optional[torch.Generator] = None) -> str:
    """src/generation.rs:205-234."""
    strategy = resolve_context_strategy(generation.context_strategy, block_size)
    prompt_ids = tokenizer.encode(generation.prompt, False, False)
    if strategy.window is not None and len(prompt_ids) > strategy.window:
        prompt_ids = prompt_ids[len(prompt_ids) - strategy.window:]
    settings = GenerationSettings(normalize_max_tokens(generation.max_tokens), generation.temperature,
                                  generation.top_k, strategy)
    tokens = generate_tokens(model, prompt_ids, settings, None, generator)
    return tokenizer.decode([t for t in tokens if t >= 0])
