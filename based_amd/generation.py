"""Generation runtime around the mixers: per-request cache bookkeeping and greedy / sampled
decoding.  Host-side mirror of based/generation.py:18-35 (InferenceParams), :64-90 (sample),
:93-204 (decode), :558-578 (GenerationMixin) and :601-739 (decode-step graph cache) of the
reference; the output container is a plain dataclass instead of the transformers classes.

The graph cache records one single-token forward of the whole stack as a HIP graph (through
torch.cuda.CUDAGraph) and replays it per token: the kernels behind the mixers take their position
from a device tensor (`lengths_per_sample`), allocate nothing outside torch's graph pool and read
nothing on the host, so a replay is one launch instead of a few hundred.
"""
from __future__ import annotations

import gc
from dataclasses import dataclass, field
from typing import Callable, Optional, Tuple

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


@dataclass
class DecodingGraphCache:
    """Captured single-token graphs of one model, keyed by (batch_size, tokens per step), with the
    pre-allocated per-layer caches they were recorded on (reference: DecodingCGCache, :601-610)."""

    max_batch_size: int = 0
    max_seqlen: int = 0
    device: Optional[torch.device] = None
    dtype: Optional[torch.dtype] = None
    callables: dict = field(default_factory=dict)
    mempool: Optional[tuple] = None
    inference_params: Optional[InferenceParams] = None
    run: Optional[Callable] = None
    # greedy decoding with the sampling inside the graph: recorded graphs keyed by (batch_size,
    # vocab_size) and the (max_batch_size, max_seqlen) buffer they write the sequences to
    greedy_graphs: dict = field(default_factory=dict)
    sequences: Optional[Tensor] = None


@torch.inference_mode()
def update_graph_cache(model, cache, batch_size, seqlen_og, max_seqlen, dtype=None, n_warmups=2, capture=True):
    """Returns a cache whose graphs fit (batch_size, max_seqlen); a larger batch, a longer
    max_seqlen or another device/dtype throws the old graphs and caches away (reference
    update_graph_cache, :613-680).  capture=False only sets up the caches (the caller records
    a graph of its own on them)."""
    if cache is None:
        cache = DecodingGraphCache()
    param = next(iter(model.parameters()))
    device = param.device
    dtype = param.dtype if dtype is None else dtype
    if ((device, dtype) != (cache.device, cache.dtype) or batch_size > cache.max_batch_size
            or max_seqlen > cache.max_seqlen):
        cache.callables = {}
        cache.greedy_graphs = {}
        cache.sequences = None
        cache.mempool = None
        cache.inference_params = None
        gc.collect()
        cache.device, cache.dtype = device, dtype
        cache.max_batch_size, cache.max_seqlen = batch_size, max_seqlen
        inf_cache = model.allocate_inference_cache(batch_size, max_seqlen, dtype)
        lengths = torch.full((batch_size,), seqlen_og, dtype=torch.int32, device=device)
        cache.inference_params = InferenceParams(max_seqlen=max_seqlen, max_batch_size=batch_size,
                                                 seqlen_offset=seqlen_og, key_value_memory_dict=inf_cache,
                                                 lengths_per_sample=lengths)
        cache.mempool = torch.cuda.graphs.graph_pool_handle()
    if capture and (batch_size, 1) not in cache.callables:
        cache.callables[batch_size, 1] = capture_graph(model, cache.inference_params, batch_size, cache.max_seqlen,
                                                       mempool=cache.mempool, n_warmups=n_warmups)

    def dispatch(input_ids, position_ids, seqlen):
        return cache.callables[input_ids.shape[0], input_ids.shape[1]](input_ids, position_ids, seqlen)

    cache.run = dispatch
    cache.inference_params.seqlen_offset = 0
    return cache


def capture_graph(model, inference_params, batch_size, max_seqlen, mempool=None, n_warmups=2):
    """Records model(one token) on static input tensors; the returned callable copies new inputs
    in, sets the device-side positions and replays (reference capture_graph, :683-739).  Warm-up
    runs on a side stream first so that lazily created buffers (workspaces, rotary tables) exist
    before the recording starts."""
    device = next(iter(model.parameters())).device
    input_ids = torch.zeros(batch_size, 1, dtype=torch.long, device=device)
    position_ids = torch.zeros(batch_size, 1, dtype=torch.long, device=device)
    offset_og = inference_params.seqlen_offset
    inference_params.seqlen_offset = max_seqlen - 1
    inference_params.lengths_per_sample[:] = max_seqlen - 1

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(n_warmups):
            logits = model(input_ids, position_ids=position_ids, inference_params=inference_params,
                           num_last_tokens=1).logits
        side.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=mempool):
        logits = model(input_ids, position_ids=position_ids, inference_params=inference_params,
                       num_last_tokens=1).logits

    def run(new_input_ids, new_position_ids, seqlen):
        inference_params.lengths_per_sample[:] = seqlen
        input_ids.copy_(new_input_ids)
        position_ids.copy_(new_position_ids)
        graph.replay()
        return logits.clone()

    inference_params.seqlen_offset = offset_og
    return run


def capture_greedy_graph(model, inference_params, sequences, batch_size, max_seqlen, vocab_size=None, mempool=None,
                         n_warmups=2):
    """Records one single-token step of the model TOGETHER with the greedy choice of the next
    token (`ops.greedy_step`): a replay reads the token in the graph's input buffer at the
    device-side position `lengths_per_sample`, and leaves the next token in that buffer and in
    `sequences`, with the positions advanced.  A decoding loop is then one replay per token and
    nothing else: no argmax kernel, no copies of ids / positions / lengths, no logits clone.
    Returns (graph, input_ids, position_ids)."""
    from . import ops

    device = next(iter(model.parameters())).device
    input_ids = torch.zeros(batch_size, 1, dtype=torch.long, device=device)
    position_ids = torch.zeros(batch_size, 1, dtype=torch.long, device=device)
    lengths = inference_params.lengths_per_sample
    seq = sequences[:batch_size]
    offset_og = inference_params.seqlen_offset
    inference_params.seqlen_offset = max_seqlen - 1

    def step():
        logits = model(input_ids, position_ids=position_ids, inference_params=inference_params,
                       num_last_tokens=1).logits.squeeze(dim=1)
        ops.greedy_step(logits, input_ids, lengths[:batch_size], sequences=seq, position_ids=position_ids,
                        vocab_size=vocab_size)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(n_warmups):
            lengths[:] = max_seqlen - 1   # (a step at the last position writes no sequence entry)
            input_ids.zero_()
            step()
        side.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    lengths[:] = max_seqlen - 1
    input_ids.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=mempool):
        step()
    inference_params.seqlen_offset = offset_og
    return graph, input_ids, position_ids


def _decode_greedy_in_graph(input_ids, model, max_length, vocab_size=None) -> DecodeOutput:
    """Greedy decoding with one graph replay per token (capture_greedy_graph); same sequences as
    `decode(..., top_k=1, cg=True)`, no scores."""
    from . import ops

    batch_size, seqlen_og = input_ids.shape
    if not hasattr(model, "_decoding_cache"):
        model._decoding_cache = None
    cache = model._decoding_cache = update_graph_cache(model, model._decoding_cache, batch_size, seqlen_og, max_length,
                                                       capture=False)
    inference_params = cache.inference_params
    inference_params.reset(max_length, batch_size)
    if cache.sequences is None:
        cache.sequences = torch.zeros(cache.max_batch_size, cache.max_seqlen, dtype=torch.long, device=input_ids.device)
    key = (batch_size, vocab_size)
    if key not in cache.greedy_graphs:
        cache.greedy_graphs[key] = capture_greedy_graph(model, inference_params, cache.sequences, batch_size,
                                                        cache.max_seqlen, vocab_size=vocab_size, mempool=cache.mempool)
    graph, step_ids, step_pos = cache.greedy_graphs[key]
    seq = cache.sequences[:batch_size]
    lengths = inference_params.lengths_per_sample[:batch_size]
    seq[:, :seqlen_og] = input_ids
    inference_params.seqlen_offset = 0
    if max_length > seqlen_og:
        logits = model(input_ids, inference_params=inference_params, num_last_tokens=1).logits[:, -1]
        inference_params.seqlen_offset = seqlen_og
        # the first new token comes from the prefill's logits; from then on the graph feeds itself
        inference_params.lengths_per_sample[:] = seqlen_og - 1
        ops.greedy_step(logits.contiguous(), step_ids, lengths, sequences=seq, position_ids=step_pos,
                        vocab_size=vocab_size)
        for _ in range(max_length - seqlen_og - 1):
            graph.replay()
        inference_params.seqlen_offset = max_length - 1
    return DecodeOutput(sequences=seq[:, :max(max_length, seqlen_og)].clone(), scores=())


@torch.inference_mode()
def decode(input_ids, model, max_length, top_k=1, top_p=0.0, temperature=1.0, eos_token_id=None,
           teacher_outputs=None, vocab_size=None, cg=False, output_scores=True, **kwargs) -> DecodeOutput:
    """Prefill on `input_ids` (batch, seq_len), then one token at a time up to max_length.
    Same control flow as the reference's `decode`; cg=True replays a recorded graph for every
    token after the prefill.  Greedy decoding under cg=True that needs no scores, no stopping
    token and no teacher tokens (output_scores=False) takes the sampling into the graph as well:
    one replay per token."""
    batch_size, seqlen_og = input_ids.shape
    teacher_len = teacher_outputs.shape[1] if teacher_outputs is not None else 0
    if (cg and top_k == 1 and not output_scores and eos_token_id is None and teacher_outputs is None
            and max_length > seqlen_og):
        return _decode_greedy_in_graph(input_ids, model, max_length, vocab_size=vocab_size)
    if cg:
        if not hasattr(model, "_decoding_cache"):
            model._decoding_cache = None
        model._decoding_cache = update_graph_cache(model, model._decoding_cache, batch_size, seqlen_og, max_length)
        inference_params = model._decoding_cache.inference_params
        inference_params.reset(max_length, batch_size)
    else:
        inference_params = InferenceParams(max_seqlen=max_length, max_batch_size=batch_size)

    def get_logits(ids):
        decoding = inference_params.seqlen_offset > 0
        position_ids = None
        if decoding:
            position_ids = torch.full((batch_size, 1), inference_params.seqlen_offset, dtype=torch.long,
                                      device=ids.device)
        if cg and decoding:
            logits = model._decoding_cache.run(ids, position_ids, inference_params.seqlen_offset).squeeze(dim=1)
        else:
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
        out = decode(input_ids, self, max_length, top_k=top_k, top_p=top_p, temperature=temperature,
                     output_scores=output_scores, **kwargs)
        if not output_scores:
            out.scores = None
        return out if return_dict_in_generate else out.sequences
