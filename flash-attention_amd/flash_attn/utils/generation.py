"""Decoding-side glue around `flash_attn_with_kvcache`: the state attention layers read while a model
generates, token selection, the token loop, and replay of one decoding step from a HIP graph.

Covers what the reference keeps in flash_attn/utils/generation.py on the attention path:
`InferenceParams` (:18-35), the top-k / top-p helpers and `sample` (:40-97), `decode` (:100-201) with
the same arguments and result type, speculative decoding (`sample_speculative`, `decode_speculative`, :204-558),
`GenerationMixin` (:561-582), and the graph cache behind `cg=True` (:604-739) with its public names
(`DecodingCGCache`, `update_graph_cache`, `capture_graph`).  A "model" is
any callable `model(input_ids, position_ids=None, inference_params=None, num_last_tokens=0)` whose
result has a `.logits` tensor of shape (batch, tokens, vocab), as the reference's GPT models do.

Why one captured step stays valid for every later step: nothing inside the attention call depends
on device values on the host (no synchronisation), its split plan is a function of the cache SHAPE,
and the kernels read the true per-sequence lengths from `lengths_per_sample`, which is rewritten on
the device before each replay.  The step is captured at the largest cache fill, so every launch in
the graph is sized for the longest sequence it will ever see.
"""
from collections import namedtuple
from dataclasses import dataclass, field
from typing import Optional

import torch
from torch import Tensor

GreedySearchDecoderOnlyOutput = namedtuple("GreedySearchDecoderOnlyOutput", ["sequences", "scores"])
SampleDecoderOnlyOutput = namedtuple("SampleDecoderOnlyOutput", ["sequences", "scores"])


@dataclass
class InferenceParams:
    """What the attention layers of a generating model share: the cache geometry, how many tokens
    every sequence already holds (`seqlen_offset`, or per sequence `lengths_per_sample`), and the
    per-layer caches `key_value_memory_dict[layer_idx]`, each
    (max_batch_size, max_seqlen, 2, nheads_kv, headdim)."""

    max_seqlen: int
    max_batch_size: int
    seqlen_offset: int = 0
    batch_size_offset: int = 0
    key_value_memory_dict: dict = field(default_factory=dict)
    lengths_per_sample: Optional[Tensor] = None

    def reset(self, max_seqlen, max_batch_size):
        self.max_seqlen, self.max_batch_size, self.seqlen_offset = max_seqlen, max_batch_size, 0
        if self.lengths_per_sample is not None:
            self.lengths_per_sample.zero_()


# ------------------------------------------------------------------------------------------------
# token selection
# ------------------------------------------------------------------------------------------------
_NEG_INF = float("-inf")


def modify_logits_for_top_k_filtering(logits, top_k):
    """In place: a row keeps its top_k largest logits, the rest become -inf."""
    smallest_kept = logits.topk(top_k, dim=-1).values[..., -1:]
    logits.masked_fill_(logits < smallest_kept, _NEG_INF)


def modify_logits_for_top_p_filtering(logits, top_p):
    """In place: the least likely tokens whose probabilities add up to at most 1 - top_p become -inf."""
    if not 0.0 < top_p < 1.0:
        return
    ascending, order = logits.sort(dim=-1)
    tail = ascending.softmax(dim=-1).cumsum(dim=-1) <= 1.0 - top_p        # in sorted order
    logits.masked_fill_(torch.zeros_like(tail).scatter_(-1, order, tail), _NEG_INF)


def _draw(logits):
    return torch.multinomial(logits.softmax(dim=-1), num_samples=1).squeeze(-1)


def sample(logits, top_k=1, top_p=0.0, temperature=1.0):
    """logits (batch, vocab) -> token ids (batch,).  top_k = 1 is greedy, top_k = 0 draws from the whole
    vocabulary; temperature and top-p apply after the top-k cut."""
    if top_k == 1:
        return logits.argmax(dim=-1)
    assert top_p <= 1.0, "top-p should be in (0, 1]."
    if top_k > 0:
        kept, ids = logits.topk(min(top_k, logits.shape[-1]), dim=-1)
        if temperature != 1.0:
            kept = kept / temperature
        modify_logits_for_top_p_filtering(kept, top_p)
        return ids.gather(-1, _draw(kept).unsqueeze(-1)).squeeze(-1)
    scaled = logits / temperature if temperature != 1.0 else logits.clone()
    modify_logits_for_top_p_filtering(scaled, top_p)
    return _draw(scaled)


def _filtered_probs(logits, top_k, top_p, temperature):
    """softmax of a copy of `logits` after temperature, the top-k cut and the top-p cut"""
    logits = logits / temperature if temperature != 1.0 else logits.clone()
    if top_k > 0:
        modify_logits_for_top_k_filtering(logits, min(top_k, logits.shape[-1]))
    modify_logits_for_top_p_filtering(logits, top_p)
    return logits.softmax(dim=-1)


def sample_speculative(logits, logits_draft, tokens_draft, top_k=1, top_p=0.0, temperature=1.0):
    """Speculative sampling (Leviathan, Kalman, Matias: Fast Inference from Transformers via Speculative
    Decoding, algorithm 1; the reference's function of the same name, flash_attn/utils/generation.py:204-262).
    logits (batch, n + 1, vocab) are the verifying model's at the n drafted positions and one more,
    logits_draft (batch, n, vocab) the drafting model's, tokens_draft (batch, n) what it drew.  A drafted token is
    kept with probability min(1, p / p_draft); the first one that is not kept is drawn again from the positive part
    of p - p_draft, and when all are kept one more token is drawn from the last position.  Returns tokens
    (batch, n + 1) and how many of them count, (batch,) values in [1, n + 1]."""
    batch, n1, vocab = logits.shape
    n = n1 - 1
    assert logits_draft.shape == (batch, n, vocab) and tokens_draft.shape == (batch, n)
    assert tokens_draft.dtype in (torch.int64, torch.int32)
    if top_p > 0.0:
        assert top_p <= 1.0, "top-p should be in (0, 1]."
    p = _filtered_probs(logits, top_k, top_p, temperature)
    q = _filtered_probs(logits_draft, top_k, top_p, temperature)
    drawn = tokens_draft.long().unsqueeze(-1)
    p_tok, q_tok = p[:, :n].gather(-1, drawn).squeeze(-1), q.gather(-1, drawn).squeeze(-1)
    kept = torch.rand(batch, n, device=p.device) * q_tok <= p_tok
    # index of the first token that is not kept, n when all are
    n_kept = torch.cat([kept, torch.zeros(batch, 1, dtype=torch.bool, device=p.device)], dim=1).int().argmin(dim=-1)
    redraw_from = torch.cat([(p[:, :n] - q).clamp_(min=0.0), p[:, n:]], dim=1)          # (batch, n + 1, vocab)
    row = redraw_from.gather(1, n_kept.view(batch, 1, 1).expand(batch, 1, vocab)).squeeze(1)
    redrawn = torch.multinomial(row, num_samples=1)                                       # unnormalised weights are fine
    tokens = torch.nn.functional.pad(tokens_draft, (0, 1)).scatter(1, n_kept.unsqueeze(1), redrawn.to(tokens_draft.dtype))
    return tokens, n_kept + 1


# ------------------------------------------------------------------------------------------------
# one decoding step as a HIP graph
# ------------------------------------------------------------------------------------------------
def allocate_inference_cache(max_batch_size, max_seqlen, nheads, headdim, layers, device, dtype=torch.float16):
    """{layer_idx: (max_batch_size, max_seqlen, 2, nheads, headdim)}; `layers` an int or an iterable."""
    assert dtype in (torch.float16, torch.bfloat16, torch.float32)
    ids = range(layers) if isinstance(layers, int) else layers
    return {i: torch.empty(max_batch_size, max_seqlen, 2, nheads, headdim, device=device, dtype=dtype) for i in ids}


class DecodeStepGraph:
    """`model` applied to (batch_size, n_tokens) new tokens against the KV caches in `state`, captured
    once and replayed.  Owns the static input buffers of the graph; the output buffer belongs to the
    graph's memory pool, so `run` hands out a copy."""

    def __init__(self, model, state: InferenceParams, batch_size, n_tokens=1, pool=None, warmups=2):
        device = next(iter(model.parameters())).device
        self.state = state
        self.tokens = torch.zeros(batch_size, n_tokens, dtype=torch.long, device=device)
        self.positions = torch.zeros(batch_size, n_tokens, dtype=torch.long, device=device)
        self.graph = torch.cuda.CUDAGraph()
        call = lambda: model(self.tokens, position_ids=self.positions, inference_params=state,
                             num_last_tokens=n_tokens).logits
        # capture at the largest fill the cache allows; the caller's fill level is put back afterwards
        fill = state.seqlen_offset
        state.seqlen_offset = state.max_seqlen - n_tokens
        state.lengths_per_sample.fill_(state.seqlen_offset)
        try:
            warm = torch.cuda.Stream()                          # default priority
            warm.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(warm):
                for _ in range(warmups):
                    call()
            warm.synchronize()
            torch.cuda.current_stream().wait_stream(warm)
            with torch.cuda.graph(self.graph, pool=pool):
                self.logits = call()
        finally:
            state.seqlen_offset = fill
            state.lengths_per_sample.fill_(fill)

    def run(self, tokens, positions, lengths):
        """lengths: an int or a (batch,) tensor: tokens every sequence holds before this step."""
        if torch.is_tensor(lengths):
            self.state.lengths_per_sample.copy_(lengths)
        else:
            self.state.lengths_per_sample.fill_(lengths)
        self.tokens.copy_(tokens)
        self.positions.copy_(positions)
        self.graph.replay()
        return self.logits.clone()


class GraphedDecoder:
    """The KV caches of one model at one geometry plus the captured steps that use them, keyed by
    (batch, new tokens per step).  All graphs share one memory pool."""

    def __init__(self, model, batch_size, max_seqlen, dtype=None, tensor_parallel=1):
        first = next(iter(model.parameters()))
        self.model, self.device, self.dtype = model, first.device, dtype or first.dtype
        self.max_batch_size, self.max_seqlen = batch_size, max_seqlen
        if hasattr(model, "allocate_inference_cache"):
            caches = model.allocate_inference_cache(batch_size, max_seqlen, self.dtype)
        else:
            cfg = model.config
            headdim = getattr(cfg, "head_dim", cfg.hidden_size // cfg.num_attention_heads)
            caches = allocate_inference_cache(batch_size, max_seqlen, cfg.num_attention_heads // tensor_parallel,
                                              headdim, cfg.num_hidden_layers, self.device, self.dtype)
        self.inference_params = InferenceParams(
            max_seqlen=max_seqlen, max_batch_size=batch_size, key_value_memory_dict=caches,
            lengths_per_sample=torch.zeros(batch_size, dtype=torch.int32, device=self.device))
        self.pool = torch.cuda.graphs.graph_pool_handle()
        self.steps = {}

    def fits(self, model, batch_size, max_seqlen, dtype=None):
        first = next(iter(model.parameters()))
        return (first.device, dtype or first.dtype) == (self.device, self.dtype) and \
            batch_size <= self.max_batch_size and max_seqlen <= self.max_seqlen

    def step(self, batch_size, n_tokens=1) -> DecodeStepGraph:
        key = (batch_size, n_tokens)
        if key not in self.steps:
            with torch.inference_mode():
                self.steps[key] = DecodeStepGraph(self.model, self.inference_params, batch_size, n_tokens, self.pool)
        return self.steps[key]

    def run(self, tokens, positions, lengths):
        return self.step(tokens.shape[0], tokens.shape[1]).run(tokens, positions, lengths)


def graphed_decoder(model, batch_size, max_seqlen, dtype=None, tensor_parallel=1) -> GraphedDecoder:
    """The model's decoder cache (kept on the model as `_decoding_cache`), rebuilt when this request
    does not fit its geometry, device or dtype."""
    dec = getattr(model, "_decoding_cache", None)
    if not isinstance(dec, GraphedDecoder) or not dec.fits(model, batch_size, max_seqlen, dtype):
        model._decoding_cache = None                 # let the old caches and graphs go first
        dec = GraphedDecoder(model, batch_size, max_seqlen, dtype, tensor_parallel)
        model._decoding_cache = dec
    return dec


# ------------------------------------------------------------------------------------------------
# the token loop
# ------------------------------------------------------------------------------------------------
class _Stepper:
    """The model behind one generation: the prompt pass, then one call per new token, eager or
    replayed from the captured step."""

    def __init__(self, model, batch_size, max_length, use_graph):
        self.model, self.batch_size = model, batch_size
        self.graphs = graphed_decoder(model, batch_size, max_length) if use_graph else None
        if use_graph:
            self.state = self.graphs.inference_params
            self.graphs.step(batch_size, 1)           # captured before the prompt pass touches the cache
            self.state.reset(max_length, batch_size)  # lengths back to 0: the prompt's rotary positions start there
        else:
            self.state = InferenceParams(max_seqlen=max_length, max_batch_size=batch_size)

    def prompt(self, input_ids):
        self.state.seqlen_offset = 0
        logits = self.model(input_ids, position_ids=None, inference_params=self.state, num_last_tokens=1).logits
        self.state.seqlen_offset = input_ids.shape[1]
        return logits[:, -1]

    def advance(self, token):
        """token (batch, 1) placed at position `seqlen_offset` of every sequence; returns its logits."""
        filled = self.state.seqlen_offset
        positions = torch.full((self.batch_size, 1), filled, dtype=torch.long, device=token.device)
        if self.graphs is not None:
            logits = self.graphs.run(token, positions, filled)
        else:
            logits = self.model(token, position_ids=positions, inference_params=self.state, num_last_tokens=1).logits
        self.state.seqlen_offset = filled + 1
        return logits[:, -1]


@torch.inference_mode()
def decode(input_ids, model, max_length, top_k=1, top_p=0.0, temperature=1.0, eos_token_id=None,
           teacher_outputs=None, vocab_size=None, tensor_parallel=1, cg=False, enable_timing=False):
    """Prompt pass over input_ids (batch, seq_len; all sequences of one length), then one token per
    step until the sequences hold max_length tokens or every sequence has just emitted eos.  With
    `teacher_outputs` (batch, len) the token at a position comes from there while it lasts, else
    from `sample`.  With `cg` every single-token step replays one captured HIP graph.  Returns
    sequences (batch, <= max_length) and the logits each new token was chosen from, a tuple of
    (batch, vocab) tensors."""
    assert tensor_parallel == 1, "one GPU: tensor parallel decoding is not part of this build"
    batch_size = input_ids.shape[0]
    taught = 0 if teacher_outputs is None else teacher_outputs.shape[1]
    stepper = _Stepper(model, batch_size, max_length, cg)
    clock = None
    if enable_timing:
        clock = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        clock[0].record()

    pieces, scores = [input_ids], []
    logits = stepper.prompt(input_ids)
    while True:
        scores.append(logits if vocab_size is None else logits[..., :vocab_size])
        at = stepper.state.seqlen_offset                       # position the next token goes to
        chosen = teacher_outputs[:, at] if at < taught else sample(scores[-1], top_k, top_p, temperature)
        pieces.append(chosen.unsqueeze(1))
        if at >= max_length - 1 or (eos_token_id is not None and bool((chosen == eos_token_id).all())):
            break
        logits = stepper.advance(pieces[-1])

    if clock is not None:
        clock[1].record()
        torch.cuda.synchronize()
        print(f"Prompt processing + decoding time: {clock[0].elapsed_time(clock[1]):.0f}ms")
    result = GreedySearchDecoderOnlyOutput if top_k == 1 else SampleDecoderOnlyOutput
    return result(sequences=torch.cat(pieces, dim=1), scores=tuple(scores))


# ------------------------------------------------------------------------------------------------
# the reference's names for the graph cache (flash_attn/utils/generation.py:605-739)
# ------------------------------------------------------------------------------------------------
DecodingCGCache = GraphedDecoder


def update_graph_cache(model, cache, batch_size, seqlen_og, max_seqlen, decoding_seqlens=(1,), tensor_parallel=1,
                       dtype=None, n_warmups=2):
    """The model's decoder cache with a captured step for every count of new tokens in `decoding_seqlens`: `cache`
    itself when it fits the request, else a new one.  `cache.run(input_ids, position_ids, seqlen)` then replays the
    step for input_ids' shape with `seqlen` tokens already cached."""
    if not isinstance(cache, GraphedDecoder) or not cache.fits(model, batch_size, max_seqlen, dtype):
        cache = None                                  # let the old caches and graphs go first
        cache = GraphedDecoder(model, batch_size, max_seqlen, dtype, tensor_parallel)
    for n_tokens in decoding_seqlens:
        cache.step(batch_size, n_tokens)
    return cache


def capture_graph(model, inference_params, batch_size, max_seqlen, decoding_seqlen=1, mempool=None, n_warmups=2):
    """One captured step of `decoding_seqlen` new tokens per sequence against the caches in `inference_params`
    (whose `lengths_per_sample` the replays read); returns run(input_ids, position_ids, seqlen) -> logits."""
    with torch.inference_mode():
        step = DecodeStepGraph(model, inference_params, batch_size, decoding_seqlen, mempool, n_warmups)
    return lambda new_input_ids, new_position_ids, seqlen: step.run(new_input_ids, new_position_ids, seqlen)


# ------------------------------------------------------------------------------------------------
# speculative decoding
# ------------------------------------------------------------------------------------------------
class _Reader:
    """A model reading one growing token sequence through its KV cache.  `seen` tokens of the sequence are in the
    cache; `read(ctx, keep)` feeds it the tokens of ctx it has not seen and returns the logits of the last `keep`
    positions fed.  Taking tokens back is setting `seen` lower: later calls overwrite the cache rows."""

    def __init__(self, model, max_length, use_graph, graph_seqlens):
        self.model = model
        self.graphs = None
        if use_graph:
            model._decoding_cache = update_graph_cache(model, getattr(model, "_decoding_cache", None), 1, 0, max_length,
                                                       decoding_seqlens=graph_seqlens)
            self.graphs = model._decoding_cache
            self.state = self.graphs.inference_params
            self.state.reset(max_length, 1)
        else:
            self.state = InferenceParams(max_seqlen=max_length, max_batch_size=1)
        self.seen = 0

    def read(self, ctx, keep=1):
        new = ctx[:, self.seen:]
        n = new.shape[1]
        assert n >= keep >= 1
        self.state.seqlen_offset = self.seen
        if self.seen == 0:
            if self.state.lengths_per_sample is not None:
                self.state.lengths_per_sample.zero_()
            logits = self.model(new, position_ids=None, inference_params=self.state, num_last_tokens=keep).logits
        else:
            positions = self.seen + torch.arange(n, dtype=torch.long, device=ctx.device).unsqueeze(0)
            if self.graphs is not None and (1, n) in self.graphs.steps:
                logits = self.graphs.run(new, positions, self.seen)[:, -keep:]
            else:
                if self.state.lengths_per_sample is not None:
                    self.state.lengths_per_sample.fill_(self.seen)
                logits = self.model(new, position_ids=positions, inference_params=self.state, num_last_tokens=keep).logits
        self.seen += n
        self.state.seqlen_offset = self.seen
        return logits


@torch.inference_mode()
def decode_speculative(input_ids, model, model_draft, max_length, speculative_lookahead=3, top_k=1, top_p=0.0,
                       temperature=1.0, eos_token_id=None, vocab_size=None, tensor_parallel=1, cg=False,
                       enable_timing=False, debug=False):
    """Speculative decoding of one sequence (batch 1, as the reference's, flash_attn/utils/generation.py:265-558):
    `model_draft` proposes up to `speculative_lookahead` tokens one by one, `model` reads them all in ONE call -- a
    few query positions against its cache, the case the KV-cache attention call packs into one row block -- and
    `sample_speculative` decides how many stand.  Greedy (top_k = 1) output is the output of `decode` with `model`
    alone.  Returns sequences (1, <= max_length) and scores (1, generated, vocab): the verifying model's logits each
    new token was taken from."""
    assert input_ids.shape[0] == 1, "Speculative decoding implementation only supports batch_size=1"
    assert eos_token_id is None, "Speculative decoding implementation doesn't support eos_token_id"
    assert tensor_parallel == 1, "one GPU: tensor parallel decoding is not part of this build"
    cut = (lambda x: x[..., :vocab_size]) if vocab_size is not None else (lambda x: x)
    main = _Reader(model, max_length, cg, range(1, speculative_lookahead + 2))
    draft = _Reader(model_draft, max_length, cg, (1, 2))
    clock = None
    if enable_timing:
        clock = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        clock[0].record()
    ctx, scores = input_ids, []
    calls = drafted = stood = 0
    while ctx.shape[1] < max_length:
        n = min(speculative_lookahead, max_length - ctx.shape[1] - 1)
        if n <= 0:                                   # room for one token: no draft
            logits = cut(main.read(ctx, 1))
            scores.append(logits)
            ctx = torch.cat([ctx, sample(logits[:, -1], top_k, top_p, temperature).unsqueeze(1)], dim=1)
            calls += 1
            break
        base = ctx.shape[1]
        proposal, logits_draft = ctx, []
        for _ in range(n):
            logits_draft.append(cut(draft.read(proposal, 1))[:, -1])
            proposal = torch.cat([proposal, sample(logits_draft[-1], top_k, top_p, temperature).unsqueeze(1)], dim=1)
        logits = cut(main.read(proposal, n + 1))                          # (1, n + 1, vocab)
        calls += 1
        tokens, counted = sample_speculative(logits, torch.stack(logits_draft, dim=1), proposal[:, base:], top_k, top_p, temperature)
        g = int(counted[0])
        drafted, stood = drafted + n, stood + g - 1
        ctx = torch.cat([ctx, tokens[:, :g]], dim=1)
        scores.append(logits[:, :g])
        # what each model has read of the new sequence: the drafts that stood (the redrawn or extra token is new to both)
        main.seen = base + g - 1
        draft.seen = min(draft.seen, base + g - 1)
        if debug:
            print("drafted %d, %d stood" % (n, g - 1))
    if clock is not None:
        clock[1].record()
        torch.cuda.synchronize()
        print(f"Prompt processing + decoding time: {clock[0].elapsed_time(clock[1]):.0f}ms")
        print(f"Number of calls to main model: {calls}")
        print(f"Acceptance rate: {100.0 * stood / max(drafted, 1):.2f}%")
    result = GreedySearchDecoderOnlyOutput if top_k == 1 else SampleDecoderOnlyOutput
    return result(sequences=ctx, scores=torch.cat(scores, dim=1))


class GenerationMixin:
    """`generate` for a model class, through `decode` (the reference's mixin, flash_attn/utils/generation.py:561-582)"""

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None, **kwargs):
        raise NotImplementedError

    def generate(self, input_ids, max_length, top_k=1, top_p=0.0, temperature=1.0, return_dict_in_generate=False,
                 output_scores=False, **kwargs):
        output = decode(input_ids, self, max_length, top_k=top_k, top_p=top_p, temperature=temperature, **kwargs)
        if not output_scores:
            output = output._replace(scores=None)
        return output if return_dict_in_generate else output.sequences
