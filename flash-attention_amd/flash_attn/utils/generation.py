"""Decoding-side glue around `flash_attn_with_kvcache`: the per-generation state that attention layers
read, the token loop, and HIP-graph capture of one decoding step.

Mirrors the parts of the reference's flash_attn/utils/generation.py that sit directly on the
attention path: `InferenceParams` (:18-35), the top-k / top-p sampling helpers (:40-97), `decode`
(:100-201), `allocate_inference_cache` (:585-601) and the graph cache (`DecodingCGCache`,
`update_graph_cache`, `capture_graph`, :604-739).  A "model" here is any callable
`model(input_ids, position_ids=None, inference_params=None, num_last_tokens=0)` that returns an
object with a `.logits` tensor of shape (batch, tokens, vocab), as the reference's GPT models do.

What makes the captured step valid: inside the attention call nothing depends on device values on
the host (no synchronisation), the split plan is a function of the cache SHAPE only, and the
per-sequence lengths are read by the kernels from `lengths_per_sample`, which `run` updates in place
before each replay.
"""
import gc
from collections import namedtuple
from dataclasses import dataclass, field
from typing import Callable, Optional

import torch
from torch import Tensor

GreedySearchDecoderOnlyOutput = namedtuple("GreedySearchDecoderOnlyOutput", ["sequences", "scores"])
SampleDecoderOnlyOutput = namedtuple("SampleDecoderOnlyOutput", ["sequences", "scores"])


@dataclass
class InferenceParams:
    """State shared by the attention layers of a model while it generates: the cache geometry, how
    many tokens every sequence already holds (`seqlen_offset`, or per sequence `lengths_per_sample`),
    and the per-layer caches `key_value_memory_dict[layer_idx]` of shape
    (max_batch_size, max_seqlen, 2, nheads_kv, headdim)."""

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


def modify_logits_for_top_k_filtering(logits, top_k):
    """In place: everything below the k-th largest logit of a row becomes -inf."""
    kth = torch.topk(logits, top_k)[0][..., -1, None]
    logits.masked_fill_(logits < kth, float("-inf"))


def modify_logits_for_top_p_filtering(logits, top_p):
    """In place: the low-probability tail whose total mass is at most 1 - top_p becomes -inf."""
    if top_p <= 0.0 or top_p >= 1.0:
        return
    sorted_logits, sorted_indices = torch.sort(logits, descending=False)
    drop_sorted = sorted_logits.softmax(dim=-1).cumsum(dim=-1) <= (1 - top_p)
    drop = drop_sorted.scatter(1, sorted_indices, drop_sorted)
    logits.masked_fill_(drop, float("-inf"))


def sample(logits, top_k=1, top_p=0.0, temperature=1.0):
    """logits (batch, vocab) -> token ids (batch,).  top_k = 1 is greedy; top_k = 0 samples from the
    whole vocabulary; top-k is applied before top-p."""
    if top_k == 1:
        return logits.argmax(dim=-1)
    if top_p > 0.0:
        assert top_p <= 1.0, "top-p should be in (0, 1]."
    if top_k > 0:
        top_k = min(top_k, logits.size(-1))
        logits_top, indices = torch.topk(logits, top_k, dim=-1)
        if temperature != 1.0:
            logits_top /= temperature
        modify_logits_for_top_p_filtering(logits_top, top_p)
        pick = torch.multinomial(torch.softmax(logits_top, dim=-1), num_samples=1).squeeze(dim=-1)
        return indices[torch.arange(indices.shape[0], device=indices.device), pick]
    logits_top = logits / temperature if temperature != 1.0 else logits.clone()
    modify_logits_for_top_p_filtering(logits_top, top_p)
    return torch.multinomial(torch.softmax(logits_top, dim=-1), num_samples=1).squeeze(dim=-1)


@torch.inference_mode()
def decode(input_ids, model, max_length, top_k=1, top_p=0.0, temperature=1.0, eos_token_id=None,
           teacher_outputs=None, vocab_size=None, tensor_parallel=1, cg=False, enable_timing=False):
    """Prompt pass, then one token per step until max_length (or every sequence emitted eos).
    input_ids (batch, seq_len), all sequences of one length.  With `teacher_outputs` (batch, len) the
    next token is taken from there instead of being sampled.  With `cg` every single-token step is
    a replay of one captured HIP graph.  Returns sequences (batch, <= max_length) and the per-step
    logits (tuple of (batch, vocab))."""
    assert tensor_parallel == 1, "one GPU: tensor parallel decoding is not part of this build"
    batch_size, seqlen_og = input_ids.shape
    teacher_len = teacher_outputs.shape[1] if teacher_outputs is not None else 0
    if cg:
        if not hasattr(model, "_decoding_cache"):
            model._decoding_cache = None
        model._decoding_cache = update_graph_cache(model, model._decoding_cache, batch_size, seqlen_og, max_length)
        inference_params = model._decoding_cache.inference_params
        inference_params.reset(max_length, batch_size)
    else:
        inference_params = InferenceParams(max_seqlen=max_length, max_batch_size=batch_size)

    def get_logits(tokens):
        decoding = inference_params.seqlen_offset > 0
        position_ids = None
        if decoding:
            position_ids = torch.full((batch_size, 1), inference_params.seqlen_offset, dtype=torch.long,
                                      device=tokens.device)
        if cg and decoding:
            logits = model._decoding_cache.run(tokens, position_ids, inference_params.seqlen_offset).squeeze(dim=1)
        else:
            logits = model(tokens, position_ids=position_ids, inference_params=inference_params,
                           num_last_tokens=1).logits.squeeze(dim=1)
        return logits[..., :vocab_size] if vocab_size is not None else logits

    def next_token(logits):
        if teacher_outputs is None or teacher_len <= inference_params.seqlen_offset:
            token = sample(logits, top_k=top_k, top_p=top_p, temperature=temperature)
        else:
            token = teacher_outputs[:, inference_params.seqlen_offset]
        return token.unsqueeze(1)

    def finished(last):
        if inference_params.seqlen_offset == 0:
            return False
        if eos_token_id is not None and (last == eos_token_id).all():
            return True
        return inference_params.seqlen_offset >= max_length - 1

    start = torch.cuda.Event(enable_timing=enable_timing)
    end = torch.cuda.Event(enable_timing=enable_timing)
    if enable_timing:
        start.record()
    scores, sequences = [], [input_ids]
    while not finished(sequences[-1]):
        scores.append(get_logits(sequences[-1]))
        inference_params.seqlen_offset += sequences[-1].shape[1]
        sequences.append(next_token(scores[-1]))
    if enable_timing:
        end.record()
        torch.cuda.synchronize()
        print(f"Prompt processing + decoding time: {(start.elapsed_time(end)):.0f}ms")
    output_cls = GreedySearchDecoderOnlyOutput if top_k == 1 else SampleDecoderOnlyOutput
    return output_cls(sequences=torch.cat(sequences, dim=1), scores=tuple(scores))


def allocate_inference_cache(max_batch_size, max_seqlen, nheads, headdim, layers, device, dtype=torch.float16):
    """{layer_idx: (max_batch_size, max_seqlen, 2, nheads, headdim)}; `layers` an int or an iterable."""
    assert dtype in (torch.float16, torch.bfloat16, torch.float32)
    if isinstance(layers, int):
        layers = range(layers)
    shape = (max_batch_size, max_seqlen, 2, nheads, headdim)
    return {i: torch.empty(shape, device=device, dtype=dtype) for i in layers}


@dataclass
class DecodingCGCache:
    max_batch_size: int = 0
    max_seqlen: int = 0
    device = None
    dtype = None
    callables: dict = field(default_factory=dict)
    mempool = None
    inference_params: Optional[InferenceParams] = None
    run: Optional[Callable] = None


@torch.inference_mode()
def update_graph_cache(model, cache, batch_size, seqlen_og, max_seqlen, decoding_seqlens=(1,), tensor_parallel=1,
                       dtype=None, n_warmups=2):
    """Make sure `cache` holds a captured step for (batch_size, each decoding_seqlen) at this cache
    geometry, (re)allocating the KV cache and `lengths_per_sample` when the geometry grew."""
    if cache is None:
        cache = DecodingCGCache()
    example = next(iter(model.parameters()))
    device = example.device
    if dtype is None:
        dtype = example.dtype
    if (device, dtype) != (cache.device, cache.dtype) or batch_size > cache.max_batch_size or max_seqlen > cache.max_seqlen:
        cache.callables = {}
        cache.mempool = None
        cache.inference_params = None
        gc.collect()
        cache.device, cache.dtype = device, dtype
        cache.max_batch_size, cache.max_seqlen = batch_size, max_seqlen
        if hasattr(model, "allocate_inference_cache"):
            kv = model.allocate_inference_cache(batch_size, max_seqlen, dtype)
        else:
            cfg = model.config
            headdim = getattr(cfg, "head_dim", cfg.hidden_size // cfg.num_attention_heads)
            kv = allocate_inference_cache(batch_size, max_seqlen, cfg.num_attention_heads // tensor_parallel, headdim,
                                          cfg.num_hidden_layers, device, dtype)
        lengths = torch.full((batch_size,), seqlen_og, dtype=torch.int32, device=device)
        cache.inference_params = InferenceParams(max_seqlen=max_seqlen, max_batch_size=batch_size, seqlen_offset=seqlen_og,
                                                 key_value_memory_dict=kv, lengths_per_sample=lengths)
        cache.mempool = torch.cuda.graphs.graph_pool_handle()
    for n in decoding_seqlens:
        if (batch_size, n) not in cache.callables:
            cache.callables[batch_size, n] = capture_graph(model, cache.inference_params, batch_size, max_seqlen,
                                                           decoding_seqlen=n, mempool=cache.mempool, n_warmups=n_warmups)

    def dispatch(input_ids, position_ids, seqlen):
        return cache.callables[input_ids.shape[0], input_ids.shape[1]](input_ids, position_ids, seqlen)

    cache.run = dispatch
    cache.inference_params.seqlen_offset = 0
    return cache


def capture_graph(model, inference_params, batch_size, max_seqlen, decoding_seqlen=1, mempool=None, n_warmups=2):
    """Capture one decoding step at the LARGEST cache fill (so that every launch is sized for it) and
    return `run(input_ids, position_ids, seqlen)`, which sets the true lengths and replays."""
    device = next(iter(model.parameters())).device
    input_ids = torch.zeros((batch_size, decoding_seqlen), dtype=torch.long, device=device)
    position_ids = torch.zeros((batch_size, decoding_seqlen), dtype=torch.long, device=device)
    offset_before = inference_params.seqlen_offset
    inference_params.seqlen_offset = max_seqlen - decoding_seqlen
    inference_params.lengths_per_sample[:] = inference_params.seqlen_offset

    side = torch.cuda.Stream()                      # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(n_warmups):
            logits = model(input_ids, position_ids=position_ids, inference_params=inference_params,
                           num_last_tokens=decoding_seqlen).logits
        side.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=mempool):
        logits = model(input_ids, position_ids=position_ids, inference_params=inference_params,
                       num_last_tokens=decoding_seqlen).logits

    def run(new_input_ids, new_position_ids, seqlen):
        inference_params.lengths_per_sample[:] = seqlen
        input_ids.copy_(new_input_ids)
        position_ids.copy_(new_position_ids)
        graph.replay()
        return logits.clone()

    inference_params.seqlen_offset = offset_before
    return run
