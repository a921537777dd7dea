"""Which workgroup computes which (batch, head, row block) is a pure scheduling choice (contiguous
eighths of the streams per XCD, every 8th stream for packed batches, groups of k streams in
unit-major order under a mask; xcd_stream_unit in csrc/fa_common.h).  Two properties pin it without
an oracle, on shapes that reach every branch of that mapping in the forward and backward kernels:

  * coverage: outputs and gradients pre-filled with NaN hold no NaN afterwards (every row of every
    stream is written by some workgroup);
  * placement: permuting the batch entries (or packed sequences) and the kv heads of the inputs
    permutes the results bit for bit (same shapes, so the same kernels and the same split plan; only
    the assignment of streams to workgroups changes).

The values themselves are pinned against the oracle by the other GPU tests."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _nat():
    from flash_attn import _native as nat
    return nat


def _nan_like(t):
    return torch.full_like(t, float("nan"))


DENSE = [
    # b, s, h, hk, d, causal, window          streams, kernel, branch
    (3, 1024, 8, 8, 64, True, (-1, -1)),     # 24 dense, 3 per XCD in one group of 3 (pipelined kernel, 96 slots)
    (5, 512, 8, 8, 128, True, (-1, -1)),     # 40, 5 per XCD in one group (pipelined kernel, 4 row blocks)
    (2, 2048, 16, 8, 128, True, (-1, -1)),   # 16, groups of 2 (ping-pong kernel, grouped q heads)
    (5, 2048, 16, 8, 128, True, (-1, -1)),   # 40, groups of 2, 2, 1: short last group
    (3, 700, 3, 3, 64, True, (-1, -1)),      # 9: not a multiple of 8, contiguous eighths of the unit order
    (2, 1024, 4, 4, 128, False, (-1, -1)),   # 8, no mask: one stream after the other
    (9, 600, 8, 8, 256, True, (-1, -1)),     # 72, head-dim-256 pair kernel
    (4, 300, 4, 2, 64, True, (100, 0)),      # 8, general kernel (fewer than 512 rows), window
    (3, 1536, 8, 8, 128, False, (200, 50)),  # 24, two-sided window on the pipelined kernel
    (1, 8192, 8, 1, 128, True, (-1, -1)),    # 1 stream: units dealt to the XCDs one by one (ping-pong kernel)
    (1, 4096, 8, 1, 128, True, (-1, -1)),    # the same with 128 blocks of 256 rows: pipelined kernel on long keys
    (2, 1024, 6, 2, 64, True, (-1, -1)),     # 4 streams, the same on the pipelined kernel
    (1, 2048, 4, 4, 128, False, (-1, -1)),   # 4 streams, no mask: contiguous eighths
]


@pytest.mark.parametrize("case", DENSE, ids=lambda c: "b%d_s%d_h%d_%d_d%d_%s" % (c[0], c[1], c[2], c[3], c[4], "m" if c[5] or c[6][0] >= 0 else "f"))
def test_dense_work_order_covers_and_places_every_stream(case):
    b, s, h, hk, d, causal, (wl, wr) = case
    _say("work order dense", case)
    nat = _nat()
    G = h // hk
    gen = torch.Generator().manual_seed(b * 1000 + s)
    q, do = (torch.randn(b, s, h, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(b, s, hk, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    scale = d ** -0.5

    def run(q, k, v, do):
        res = nat.fwd(q, k, v, _nan_like(q), 0.0, scale, causal, wl, wr, False, None)
        out, lse = res[0], res[5]
        dq, dk, dv = _nan_like(q), _nan_like(k), _nan_like(v)
        nat.bwd(do, q, k, v, out, lse, dq, dk, dv, 0.0, scale, causal, wl, wr, None, None)
        for name, t in (("out", out), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
            assert not torch.isnan(t).any(), "%s has rows no workgroup wrote" % name
        return out, lse, dq, dk, dv

    out, lse, dq, dk, dv = run(q, k, v, do)
    pb = torch.randperm(b, generator=gen).to(DEV)
    ph = torch.randperm(hk, generator=gen)
    qh = (ph[:, None] * G + torch.arange(G)[None]).flatten().to(DEV)
    ph = ph.to(DEV)
    perm_q = lambda t: t[pb][:, :, qh].contiguous()
    perm_k = lambda t: t[pb][:, :, ph].contiguous()
    out2, lse2, dq2, dk2, dv2 = run(perm_q(q), perm_k(k), perm_k(v), perm_q(do))
    assert torch.equal(out2, perm_q(out))
    assert torch.equal(lse2, lse[pb][:, qh])
    assert torch.equal(dq2, perm_q(dq))
    assert torch.equal(dk2, perm_k(dk)) and torch.equal(dv2, perm_k(dv))


PACKED = [
    # lengths, h, hk, d, causal
    ([900, 130, 1500, 64, 700, 1024, 333, 1200, 512], 8, 8, 128, True),   # 72 streams, every 8th, groups
    ([1100, 40, 513, 777, 260], 4, 2, 64, True),                           # 10: XCDs hold 2 or 1 streams
    ([600, 1030, 90], 4, 2, 128, True),                                    # 6 < 8: contiguous eighths
    ([2300, 150, 2048, 900, 1700, 31, 1, 640], 2, 1, 128, True),           # 8 streams, ping-pong kernel
    ([700, 520, 64, 900, 1300, 200, 1024, 45], 8, 8, 256, False),          # pair kernel, no mask
    ([900, 130, 1500, 64, 700, 1024, 333, 1200, 512], 8, 1, 128, True),   # MQA: the 8 q heads of a stream go to 8 XCDs (forward)
    ([1100, 40, 513, 777, 260, 2100], 8, 2, 64, True),                     # GQA: 2 kv heads x 4 parts of 1 q head (forward)
    ([600, 1030, 90, 300], 12, 2, 128, True),                              # 6 q heads per kv head: not cut
]


@pytest.mark.parametrize("case", PACKED, ids=lambda c: "n%d_h%d_%d_d%d_%s" % (len(c[0]), c[1], c[2], c[3], "m" if c[4] else "f"))
def test_packed_work_order_covers_and_places_every_stream(case):
    lens, h, hk, d, causal = case
    _say("work order packed", case)
    nat = _nat()
    n, G, mx, total = len(lens), h // hk, max(lens), sum(lens)
    gen = torch.Generator().manual_seed(n * 100 + d)
    q, do = (torch.randn(total, h, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    k, v = (torch.randn(total, hk, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    scale = d ** -0.5

    def cu_of(ls):
        return torch.tensor([0] + ls).cumsum(0).to(torch.int32)

    def run(q, k, v, do, ls):
        cu = cu_of(ls).to(DEV)
        res = nat.varlen_fwd(q, k, v, _nan_like(q), cu, cu, mx, mx, 0.0, scale, False, causal, -1, -1, False, None)
        out, lse = res[0], res[5]
        dq, dk, dv = _nan_like(q), _nan_like(k), _nan_like(v)
        nat.varlen_bwd(do, q, k, v, out, lse, dq, dk, dv, cu, cu, mx, mx, 0.0, scale, False, causal, -1, -1, None, None)
        for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
            assert not torch.isnan(t).any(), "%s has rows no workgroup wrote" % name
        return out, lse, dq, dk, dv

    out, lse, dq, dk, dv = run(q, k, v, do, lens)
    ps = torch.randperm(n, generator=gen).tolist()
    ph = torch.randperm(hk, generator=gen)
    qh = (ph[:, None] * G + torch.arange(G)[None]).flatten().to(DEV)
    ph = ph.to(DEV)
    cu = cu_of(lens).tolist()
    rows = torch.cat([torch.arange(cu[i], cu[i + 1]) for i in ps]).to(DEV)        # packed rows in the new order
    perm_q = lambda t: t[rows][:, qh].contiguous()
    perm_k = lambda t: t[rows][:, ph].contiguous()
    lens2 = [lens[i] for i in ps]
    out2, lse2, dq2, dk2, dv2 = run(perm_q(q), perm_k(k), perm_k(v), perm_q(do), lens2)
    assert torch.equal(out2, perm_q(out))
    assert torch.equal(dq2, perm_q(dq))
    assert torch.equal(dk2, perm_k(dk)) and torch.equal(dv2, perm_k(dv))
    for j, i in enumerate(ps):       # log-sum-exp is (sequence, head, max_seqlen); rows past a length are unwritten
        assert torch.equal(lse2[j][:, : lens[i]], lse[i][qh][:, : lens[i]])
