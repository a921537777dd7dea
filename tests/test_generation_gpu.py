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
    multiple of 16 (the standalone kernel's granule) and must be rejected with a clear error."""
    from flash_attn.modules.mha import MHA
    _say("mha layer", heads_kv, rotary_dim)
    torch.manual_seed(1)
    dtype, b, s, dim, h = torch.float16, 2, 150, 256, 4
    d = dim // h
    layer = MHA(dim, h, num_heads_kv=heads_kv, causal=True, layer_idx=0, rotary_emb_dim=rotary_dim, device=DEV, dtype=dtype)
    x = torch.randn(b, s, dim, device=DEV, dtype=dtype)
    if rotary_dim == 24:
        with pytest.raises(RuntimeError, match="divisible by 16"):
            layer(x)
        return
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
@pytest.mark.parametrize("rotary_dim", [0, 32])
def test_incremental_decoding_matches_full_forward(heads_kv, rotary_dim):
    """Teacher-forced decode: logits of step t from the cache paths (prompt pass, then the fused
    rotary + append + attend call per token) against one full forward over the whole sequence."""
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
