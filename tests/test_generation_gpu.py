"""GPU tests of the decoding glue: the MHA layer's cache paths and the token loop, eager and as replays
of a captured HIP graph.  The strategy is the reference's for generation (tests/models/test_gpt.py,
test_gpt_generation: incremental decoding must reproduce a full forward over the same tokens, and the
graph-captured loop must reproduce the eager loop), on a two-layer toy model so that the attention
path is the only thing under test.  The full forward itself is checked against the CPU oracle."""
import sys
from types import SimpleNamespace

import pytest
import torch
import torch.nn as nn

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


class ToyLM(nn.Module):
    """embedding -> n x (x + MHA(x)) -> vocabulary projection; the call contract of the reference's
    GPT models (`position_ids`, `inference_params`, `num_last_tokens`, result with `.logits`)."""

    def __init__(self, vocab, dim, heads, heads_kv, layers, rotary_dim, dtype):
        super().__init__()
        from flash_attn.modules.mha import MHA
        self.emb = nn.Embedding(vocab, dim, device=DEV, dtype=dtype)
        self.layers = nn.ModuleList([
            MHA(dim, heads, num_heads_kv=heads_kv, causal=True, layer_idx=i, rotary_emb_dim=rotary_dim,
                rotary_emb_interleaved=(i % 2 == 1), device=DEV, dtype=dtype) for i in range(layers)])
        self.head = nn.Linear(dim, vocab, bias=False, device=DEV, dtype=dtype)

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None):
        return {i: l.allocate_inference_cache(batch_size, max_seqlen, dtype) for i, l in enumerate(self.layers)}

    def forward(self, input_ids, position_ids=None, inference_params=None, num_last_tokens=0):
        x = self.emb(input_ids)
        for l in self.layers:
            x = x + l(x, inference_params=inference_params)
        if num_last_tokens > 0:
            x = x[:, -num_last_tokens:]
        return SimpleNamespace(logits=self.head(x))


def _model(heads_kv, rotary_dim, dtype=torch.float16, seed=0):
    torch.manual_seed(seed)
    return ToyLM(vocab=211, dim=256, heads=4, heads_kv=heads_kv, layers=2, rotary_dim=rotary_dim, dtype=dtype).eval()


@pytest.mark.parametrize("heads_kv", [4, 1])
@pytest.mark.parametrize("rotary_dim", [0, 32, 24])
def test_mha_layer_matches_oracle(heads_kv, rotary_dim):
    """One layer, no cache: projection in torch, rotary + causal attention through the package; the
    same computed with the oracle's rotary and attention on the CPU.  rotary_dim = 24 is not a
    multiple of 16 (the granule of the memory-bound rotary kernel): the element-wise kernel takes it."""
    from flash_attn.modules.mha import MHA
    _say("mha layer", heads_kv, rotary_dim)
    torch.manual_seed(1)
    dtype, b, s, dim, h = torch.float16, 2, 150, 256, 4
    d = dim // h
    layer = MHA(dim, h, num_heads_kv=heads_kv, causal=True, layer_idx=0, rotary_emb_dim=rotary_dim, device=DEV, dtype=dtype)
    x = torch.randn(b, s, dim, device=DEV, dtype=dtype)
    with torch.no_grad():
        got = layer(x)
        qkv = layer.Wqkv(x).cpu()
    q = qkv[..., : h * d].reshape(b, s, h, d)
    k = qkv[..., h * d: (h + heads_kv) * d].reshape(b, s, heads_kv, d)
    v = qkv[..., (h + heads_kv) * d:].reshape(b, s, heads_kv, d)
    if rotary_dim:
        cos, sin = layer.rotary_emb._cos_cached.cpu(), layer.rotary_emb._sin_cached.cpu()
        pos = torch.arange(s)[None].expand(b, s)
        q, k = orc.rotary_apply(q, cos, sin, pos, False), orc.rotary_apply(k, cos, sin, pos, False)
    ctx, _ = orc.attention_forward(q, k, v, causal=True)
    want = torch.nn.functional.linear(ctx.reshape(b, s, dim).float(), layer.out_proj.weight.float().cpu(),
                                      layer.out_proj.bias.float().cpu())
    err = (got.float().cpu() - want).abs().max().item()
    _say("   err %.3e" % err)
    assert err < 5e-3


@pytest.mark.parametrize("heads_kv", [4, 2])
@pytest.mark.parametrize("rotary_dim", [0, 32, 24])
def test_incremental_decoding_matches_full_forward(heads_kv, rotary_dim):
    """Teacher-forced decode: logits of step t from the cache paths (prompt pass, then the fused
    rotary + append + attend call per token; rotary dimension 24, which that call does not rotate, goes through
    the stand-alone rotary op at each sequence's length) against one full forward over the whole sequence."""
    from flash_attn.utils.generation import decode
    _say("incremental", heads_kv, rotary_dim)
    model = _model(heads_kv, rotary_dim)
    g = torch.Generator().manual_seed(2)
    b, prompt, total = 3, 37, 70
    tokens = torch.randint(0, 211, (b, total), generator=g).to(DEV)
    with torch.no_grad():
        full = model(tokens).logits.float()
    out = decode(tokens[:, :prompt], model, total, teacher_outputs=tokens)
    assert torch.equal(out.sequences, tokens)
    assert len(out.scores) == total - prompt
    for i, step_logits in enumerate(out.scores):
        ref = full[:, prompt - 1 + i]
        err = (step_logits.float() - ref).abs().max().item()
        assert err < 2e-2 * max(1.0, ref.abs().max().item()), "step %d: %g" % (i, err)


@pytest.mark.parametrize("heads_kv", [4, 1])
def test_graph_captured_decoding_matches_eager(heads_kv):
    """The same token loop with every single-token step replayed from one captured HIP graph: captured
    at the largest cache fill, replayed at the true lengths through `lengths_per_sample`.  Several
    replays with eager work and synchronisations in between; every step's logits are compared."""
    from flash_attn.utils.generation import decode
    _say("graph decode", heads_kv)
    model = _model(heads_kv, 32)
    g = torch.Generator().manual_seed(3)
    b, prompt, total = 4, 20, 60
    tokens = torch.randint(0, 211, (b, total), generator=g).to(DEV)
    eager = decode(tokens[:, :prompt], model, total, teacher_outputs=tokens)
    torch.cuda.synchronize()
    for rep in range(2):                         # second pass reuses the captured graph
        cg = decode(tokens[:, :prompt], model, total, teacher_outputs=tokens, cg=True)
        torch.cuda.synchronize()
        assert torch.equal(cg.sequences, eager.sequences)
        for i, (a, c) in enumerate(zip(cg.scores, eager.scores)):
            err = (a.float() - c.float()).abs().max().item()
            assert err < 1e-2 * max(1.0, c.float().abs().max().item()), "pass %d step %d: %g" % (rep, i, err)
    # free-running greedy generation agrees as well (same argmax at every step)
    free_e = decode(tokens[:, :prompt], model, total)
    free_g = decode(tokens[:, :prompt], model, total, cg=True)
    assert torch.equal(free_e.sequences, free_g.sequences)


def test_sampling_helpers():
    from flash_attn.utils.generation import modify_logits_for_top_k_filtering, modify_logits_for_top_p_filtering, sample
    logits = torch.tensor([[0.0, 1.0, 2.0, 3.0], [3.0, 2.0, 1.0, 0.0]], device=DEV)
    assert sample(logits).tolist() == [3, 0]
    x = logits.clone(); modify_logits_for_top_k_filtering(x, 2)
    assert torch.isinf(x).sum().item() == 4 and x[0, 3] == 3.0 and x[1, 1] == 2.0
    x = logits.clone(); modify_logits_for_top_p_filtering(x, 0.5)      # keeps the head of the distribution
    assert x[0, 3] == 3.0 and torch.isinf(x[0, 0])
    torch.manual_seed(0)
    picks = torch.stack([sample(logits, top_k=2, top_p=0.0, temperature=0.7) for _ in range(50)])
    assert set(picks[:, 0].tolist()) <= {2, 3} and set(picks[:, 1].tolist()) <= {0, 1}


@pytest.mark.parametrize("heads_kv", [4, 2])
@pytest.mark.parametrize("rotary_dim", [0, 32])
def test_mha_packed_varlen_equals_per_sequence(heads_kv, rotary_dim):
    """Packed (total, dim) input with cu_seqlens: every sequence must come out as if it went through the
    layer alone (rotary positions restart at 0 for each sequence)."""
    from flash_attn.modules.mha import MHA
    _say("mha varlen", heads_kv, rotary_dim)
    torch.manual_seed(5)
    dtype, dim, h = torch.bfloat16, 256, 4
    layer = MHA(dim, h, num_heads_kv=heads_kv, causal=True, layer_idx=0, rotary_emb_dim=rotary_dim, device=DEV, dtype=dtype).eval()
    lens = [70, 1, 200, 33]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    x = torch.randn(sum(lens), dim, device=DEV, dtype=dtype)
    with torch.no_grad():
        packed = layer(x, cu_seqlens=cu, max_seqlen=max(lens))
        for i, L in enumerate(lens):
            a, e = int(cu[i]), int(cu[i + 1])
            alone = layer(x[a:e][None])[0]
            err = (packed[a:e].float() - alone.float()).abs().max().item()
            assert err < 2e-2, (i, err)


@pytest.mark.parametrize("heads_kv", [4, 2])
def test_mha_packed_varlen_rotary_gradients(heads_kv):
    """Training through the packed path with rotary: the gradients of the projection weights must be
    those of the same sequences sent through the layer one at a time (the rotation's backward has to
    run for the q and k parts of Wqkv)."""
    from flash_attn.modules.mha import MHA
    _say("mha varlen grad", heads_kv)
    torch.manual_seed(7)
    dtype, dim, h = torch.bfloat16, 256, 4
    layer = MHA(dim, h, num_heads_kv=heads_kv, causal=True, layer_idx=0, rotary_emb_dim=32, device=DEV, dtype=dtype)
    lens = [70, 1, 200, 33]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    x = torch.randn(sum(lens), dim, device=DEV, dtype=dtype)
    w = torch.randn(sum(lens), dim, device=DEV, dtype=dtype)

    def grads(run):
        layer.zero_grad(set_to_none=True)
        (run().float() * w.float()).sum().backward()
        return layer.Wqkv.weight.grad.float().clone(), layer.out_proj.weight.grad.float().clone()

    g_packed = grads(lambda: layer(x, cu_seqlens=cu, max_seqlen=max(lens)))
    g_alone = grads(lambda: torch.cat([layer(x[int(cu[i]):int(cu[i + 1])][None])[0] for i in range(len(lens))]))
    for name, a, b in zip(("Wqkv", "out_proj"), g_packed, g_alone):
        err = (a - b).abs().max().item()
        _say("   %s grad: max diff %.3e of max %.3e" % (name, err, b.abs().max().item()))
        assert err <= 2e-2 * b.abs().max().item(), (name, err)
    # the q and k rows of Wqkv are the ones an in-place rotation without backward would get wrong
    d = dim // h
    qk_rows = slice(0, (h + heads_kv) * d)
    assert (g_packed[0][qk_rows] - g_alone[0][qk_rows]).abs().max().item() <= 2e-2 * g_alone[0][qk_rows].abs().max().item()


def test_flash_attention_wrappers_train_and_eval():
    """FlashSelfAttention / FlashCrossAttention: dropout only in training mode, gradients flow, the
    eval output equals the functional call."""
    import flash_attn
    from flash_attn.modules.mha import FlashCrossAttention, FlashSelfAttention
    _say("wrappers")
    torch.manual_seed(6)
    qkv = torch.randn(2, 130, 3, 4, 64, device=DEV, dtype=torch.float16, requires_grad=True)
    sa = FlashSelfAttention(causal=True, attention_dropout=0.3)
    sa.eval()
    assert torch.equal(sa(qkv), flash_attn.flash_attn_qkvpacked_func(qkv, causal=True))
    sa.train()
    torch.cuda.manual_seed(1)
    out_a = sa(qkv)
    torch.cuda.manual_seed(1)
    out_b = sa(qkv)
    assert torch.equal(out_a, out_b) and not torch.equal(out_a, sa.eval()(qkv))
    out_a.float().sum().backward()
    assert qkv.grad is not None and torch.isfinite(qkv.grad).all()
    q = torch.randn(2, 50, 4, 64, device=DEV, dtype=torch.float16)
    kv = torch.randn(2, 90, 2, 2, 64, device=DEV, dtype=torch.float16)
    ca = FlashCrossAttention().eval()
    assert torch.equal(ca(q, kv), flash_attn.flash_attn_kvpacked_func(q, kv))
    cu_q = torch.tensor([0, 50, 100], dtype=torch.int32, device=DEV)
    cu_k = torch.tensor([0, 90, 180], dtype=torch.int32, device=DEV)
    packed = ca(q.reshape(100, 4, 64), kv.reshape(180, 2, 2, 64), cu_seqlens=cu_q, max_seqlen=50, cu_seqlens_k=cu_k,
                max_seqlen_k=90)
    assert (packed.reshape(2, 50, 4, 64).float() - ca(q, kv).float()).abs().max().item() < 2e-3


def test_mha_trains_with_dropout():
    """Forward + backward through the layer in training mode (attention dropout on): finite gradients for
    every parameter, and the same seed reproduces them."""
    from flash_attn.modules.mha import MHA
    _say("mha train")
    torch.manual_seed(7)
    layer = MHA(256, 4, num_heads_kv=2, dropout=0.1, causal=True, rotary_emb_dim=32, device=DEV, dtype=torch.bfloat16).train()
    x = torch.randn(2, 300, 256, device=DEV, dtype=torch.bfloat16)
    grads = []
    for _ in range(2):
        layer.zero_grad()
        torch.cuda.manual_seed(11)
        layer(x).float().square().mean().backward()
        grads.append([p.grad.clone() for p in layer.parameters()])
    for a, b in zip(*grads):
        assert torch.isfinite(a).all() and torch.equal(a, b)


@pytest.mark.parametrize("cg", [False, True])
@pytest.mark.parametrize("same_draft", [False, True])
@pytest.mark.parametrize("heads_kv,rotary_dim", [(4, 32), (1, 0)])
def test_speculative_decoding_reproduces_greedy_decoding(heads_kv, rotary_dim, same_draft, cg):
    """Greedy speculative decoding must give the verifying model's own greedy continuation, whatever the drafting
    model proposes (a different random model: most drafts are thrown away; the model itself: all stand and every
    call of the verifier reads lookahead + 1 positions against its cache, the few-positions form of the KV-cache
    attention call).  With cg the single- and multi-token steps replay captured graphs."""
    from flash_attn.utils.generation import decode, decode_speculative
    _say("speculative", heads_kv, rotary_dim, same_draft, cg)
    model = _model(heads_kv, rotary_dim)
    draft = model if same_draft else _model(heads_kv, rotary_dim, seed=5)
    g = torch.Generator().manual_seed(4)
    prompt, total = 19, 60
    ids = torch.randint(0, 211, (1, prompt), generator=g).to(DEV)
    plain = decode(ids, model, total)
    for lookahead in (1, 3, 4):
        spec = decode_speculative(ids, model, draft, total, speculative_lookahead=lookahead, cg=cg)
        assert spec.sequences.shape == (1, total)
        # positions where the plain run's top two logits are closer than the error between one-token and
        # several-token evaluation may legitimately differ; everything up to the first such position must agree
        gaps = torch.stack([s.float().topk(2, dim=-1).values for s in plain.scores], 1)[0]
        close = ((gaps[:, 0] - gaps[:, 1]) < 2e-2).nonzero()
        upto = total if close.numel() == 0 else prompt + int(close[0])
        assert torch.equal(spec.sequences[:, :upto], plain.sequences[:, :upto]), lookahead
        assert spec.scores.shape[:2] == (1, total - prompt)
        if upto == total:
            ref = torch.stack(list(plain.scores), 1).float()
            assert (spec.scores.float() - ref).abs().max().item() < 2e-2 * max(1.0, ref.abs().max().item())


def test_generation_mixin_and_graph_cache_names():
    """`GenerationMixin.generate`, `update_graph_cache` / `DecodingCGCache` / `capture_graph` as the reference names
    them (flash_attn/utils/generation.py:561-582, 605-739)."""
    from flash_attn.utils import generation as gen

    class Mixed(ToyLM, gen.GenerationMixin):
        pass
    torch.manual_seed(0)
    model = Mixed(vocab=211, dim=256, heads=4, heads_kv=2, layers=2, rotary_dim=32, dtype=torch.float16).eval()
    ids = torch.randint(0, 211, (2, 11), generator=torch.Generator().manual_seed(1)).to(DEV)
    seqs = model.generate(ids, 30)
    assert torch.is_tensor(seqs) and seqs.shape == (2, 30) and torch.equal(seqs[:, :11], ids)
    out = model.generate(ids, 30, return_dict_in_generate=True, output_scores=True)
    assert torch.equal(out.sequences, seqs) and len(out.scores) == 19
    assert model.generate(ids, 30, return_dict_in_generate=True).scores is None
    graphed = model.generate(ids, 30, cg=True)
    assert torch.equal(graphed, seqs)
    cache = gen.update_graph_cache(model, None, 2, 11, 40, decoding_seqlens=(1, 3))
    assert isinstance(cache, gen.DecodingCGCache) and set(cache.steps) == {(2, 1), (2, 3)}
    assert gen.update_graph_cache(model, cache, 2, 11, 40) is cache             # fits: kept
    assert gen.update_graph_cache(model, cache, 2, 11, 80) is not cache         # longer sequences: rebuilt
    # a captured three-token step against an eager one on the same cache contents
    state = cache.inference_params
    with torch.inference_mode():
        state.reset(40, 2)
        model(ids, inference_params=state, num_last_tokens=1)
        state.seqlen_offset = 11
        new = torch.randint(0, 211, (2, 3), generator=torch.Generator().manual_seed(2)).to(DEV)
        pos = 11 + torch.arange(3, device=DEV).expand(2, 3)
        replayed = cache.run(new, pos, 11)
        state.lengths_per_sample.fill_(11)
        eager = model(new, position_ids=pos, inference_params=state, num_last_tokens=3).logits
        assert (replayed.float() - eager.float()).abs().max().item() < 2e-2
        run = gen.capture_graph(model, state, 2, 40, decoding_seqlen=3, mempool=cache.pool)
        assert (run(new, pos, 11).float() - eager.float()).abs().max().item() < 2e-2
