"""fa_fwd_kvcache_noalloc against fa_fwd_kvcache through the C ABI: the entry point that keeps its split
accumulators and ticket words in the library's own device array must give the same output,
log-sum-exp and cache contents, bit for bit (the split plan and the merge order are the same and no
result depends on which workgroup draws which ticket), on two calls in a row that share the array,
the second with a smaller problem; oversized problems are rejected with an error."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _case(nat, b, cap, h, hk, d, lens, seqlen_q=1, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)
    kc, vc = mk(b, cap, hk, d), mk(b, cap, hk, d)
    q, kn, vn = mk(b, seqlen_q, h, d), mk(b, seqlen_q, hk, d), mk(b, seqlen_q, hk, d)
    ang = torch.outer(torch.arange(cap, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d)))
    cos, sin = torch.cos(ang).to(torch.bfloat16).to(DEV), torch.sin(ang).to(torch.bfloat16).to(DEV)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=DEV)
    results = []
    for no_alloc in (False, True):
        kc_i, vc_i = kc.clone(), vc.clone()
        out = torch.full((b, seqlen_q, h, d), float("nan"), dtype=torch.bfloat16, device=DEV)
        lse = torch.full((b, h, seqlen_q), float("nan"), dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        o, l = nat.fwd_kvcache(q, kc_i, vc_i, kn, vn, lens_d, cos, sin, None, out, d ** -0.5, True, -1, -1, True, 0,
                               no_alloc=no_alloc, lse_=lse)
        after = torch.cuda.memory_stats()["allocation.all.allocated"]
        torch.cuda.synchronize()
        if no_alloc:
            assert after == before, "the no-allocation call asked torch for device memory"
        assert o.data_ptr() == out.data_ptr() and l.data_ptr() == lse.data_ptr()
        results.append((out, lse, kc_i, vc_i))
    (o0, l0, k0, v0), (o1, l1, k1, v1) = results
    assert not torch.isnan(o1).any() and not torch.isnan(l1).any()
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    assert torch.equal(k0, k1) and torch.equal(v0, v1)


def test_no_alloc_entry_matches_kvcache_entry_twice():
    import flash_attn._native as nat
    _say("no_alloc first call: 8 x 32768 x 16 x 64 (persistent decode kernel + merge)")
    _case(nat, 8, 32768, 16, 16, 64, [32767, 1100, 3000, 5, 0, 20000, 1024, 2047], seed=1)
    _say("no_alloc second call, smaller: 3 x 5000 x 2 x 128 (one workgroup per chunk + merge)")
    _case(nat, 3, 5000, 16, 2, 128, [4999, 0, 1234], seed=2)
    _say("no_alloc third call: 2 query rows, unsplit")
    _case(nat, 2, 300, 4, 2, 64, [100, 299 - 2], seqlen_q=2, seed=3)
    _say("no_alloc fourth call: 4 query positions x 8 grouped heads (tiled kernel under the ticket schedule + merge)")
    _case(nat, 3, 9000, 32, 4, 128, [8700, 40, 4100], seqlen_q=4, seed=4)


def test_no_alloc_entry_rejects_what_does_not_fit():
    import ctypes
    import flash_attn._native as nat
    _say("no_alloc too large")
    # batch 64 x 64 heads x 40 rows x 32 splits of fp32 partials is far beyond the array
    b, cap, h, hk, d, sq = 64, 8192, 64, 8, 128, 40
    q = torch.zeros(b, sq, h, d, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(b, cap, hk, d, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="FA_NOALLOC_SCRATCH_BYTES"):
        nat.fwd_kvcache(q, kc, kc, None, None, None, None, None, None, None, d ** -0.5, True, -1, -1, True, 32, no_alloc=True)
    # the same problem unsplit needs no partials and is accepted
    out, lse = nat.fwd_kvcache(q, kc, kc, None, None, None, None, None, None, None, d ** -0.5, True, -1, -1, True, 1, no_alloc=True)
    torch.cuda.synchronize()
    assert torch.isfinite(lse).all()
