"""Generation runtime around the mixers: per-request cache bookkeeping and greedy / sampled
decoding.  Host-side mirror of based/generation.py:18-35 (InferenceParams), :64-90 (sample),
:93-204 (decode) and :558-578 (GenerationMixin) of the reference; the output container is a
plain dataclass instead of the transformers classes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple

import torch
from torch import Tensor


@dataclass
class InferenceParams:
    """Inference parameters passed down to the mixers so that they can store and find their
    per-layer caches (field-for-field the reference's container)."""

    max_seqlen: int
    max_batch_size: int
    seqlen_offset: int = 0
    batch_size_offset: int = 0
    key_value_memory_dict: dict = field(default_factory=dict)
    lengths_per_sample: Optional[Tensor] = None

    def reset(self, max_seqlen, max_batch_size):
        self.max_seqlen = max_seqlen
        self.max_batch_size = max_batch_size
        self.seqlen_offset = 0
        if self.lengths_per_sample is not None:
            self.lengths_per_sample.zero_()


@dataclass
class DecodeOutput:
    sequences: Tensor            # (batch, max_length)
    scores: Tuple[Tensor, ...]   # one (batch, vocab) tensor per generated position


def _top_p_filter_(logits: Tensor, top_p: float) -> None:
    if top_p <= 0.0 or top_p >= 1.0:
        return
    sorted_logits, sorted_idx = torch.sort(logits, descending=False)
    cum = sorted_logits.softmax(dim=-1).cumsum(dim=-1)
    drop_sorted = cum <= (1 - top_p)
    drop = drop_sorted.scatter(1, sorted_idx, drop_sorted)
    logits.masked_fill_(drop, float("-inf"))


def sample(logits: Tensor, top_k: int = 1, top_p: float = 0.0, temperature: float = 1.0) -> Tensor:
    """logits (batch, vocab) -> token ids (batch,).  top_k == 1 is greedy."""
    if top_k == 1:
        return logits.argmax(dim=-1)
    if top_p > 0.0:
        assert top_p <= 1.0, "top-p should be in (0, 1]."
    if top_k > 0:
        top_k = min(top_k, logits.size(-1))
        logits_top, indices = torch.topk(logits, top_k, dim=-1)
        if temperature != 1.0:
            logits_top = logits_top / temperature
        _top_p_filter_(logits_top, top_p)
        pick = torch.multinomial(torch.softmax(logits_top, dim=-1), num_samples=1).squeeze(-1)
        return indices[torch.arange(indices.shape[0], device=indices.device), pick]
    logits_top = logits / temperature if temperature != 1.0 else logits.clone()
    _top_p_filter_(logits_top, top_p)
    return torch.multinomial(torch.softmax(logits_top, dim=-1), num_samples=1).squeeze(-1)


@torch.inference_mode()
def decode(input_ids, model, max_length, top_k=1, top_p=0.0, temperature=1.0, eos_token_id=None,
           teacher_outputs=None, vocab_size=None, **kwargs) -> DecodeOutput:
    """Prefill on `input_ids` (batch, seq_len), then one token at a time up to max_length.
    Same control flow as the reference's `decode` without the CUDA-graph branch."""
    batch_size, _ = input_ids.shape
    teacher_len = teacher_outputs.shape[1] if teacher_outputs is not None else 0
    inference_params = InferenceParams(max_seqlen=max_length, max_batch_size=batch_size)

    def get_logits(ids):
        decoding = inference_params.seqlen_offset > 0
        position_ids = None
        if decoding:
            position_ids = torch.full((batch_size, 1), inference_params.seqlen_offset, dtype=torch.long,
                                      device=ids.device)
        logits = model(ids, position_ids=position_ids, inference_params=inference_params,
                       num_last_tokens=1).logits.squeeze(dim=1)
        return logits[..., :vocab_size] if vocab_size is not None else logits

    def next_token(logits):
        if teacher_outputs is None or teacher_len <= inference_params.seqlen_offset:
            tok = sample(logits, top_k=top_k, top_p=top_p, temperature=temperature)
        else:
            tok = teacher_outputs[:, inference_params.seqlen_offset]
        return tok.unsqueeze(1)

    def should_stop(tok):
        if inference_params.seqlen_offset == 0:
            return False
        if eos_token_id is not None and (tok == eos_token_id).all():
            return True
        return inference_params.seqlen_offset >= max_length - 1

    scores, sequences = [], [input_ids]
    while not should_stop(sequences[-1]):
        scores.append(get_logits(sequences[-1]))
        inference_params.seqlen_offset += sequences[-1].shape[1]
        sequences.append(next_token(scores[-1]))
    return DecodeOutput(sequences=torch.cat(sequences, dim=1), scores=tuple(scores))


class GenerationMixin:
    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None, **kwargs):
        raise NotImplementedError

    def generate(self, input_ids, max_length, top_k=1, top_p=0.0, temperature=1.0,
                 return_dict_in_generate=False, output_scores=False, **kwargs):
        out = decode(input_ids, self, max_length, top_k=top_k, top_p=top_p, temperature=temperature, **kwargs)
        if not output_scores:
            out.scores = None
        return out if return_dict_in_generate else out.sequences
