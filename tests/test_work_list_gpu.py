"""Packed (variable-length) forward launches walk a work list that the library builds on the device from
cu_seqlens_q (work_list_kernel, csrc/fa_aux.hip) when the caller lends it fa_work_list_words() words.  The
list only changes which workgroup computes which row block: every output row must be written, and the
results must equal those of the arithmetic work order bit for bit."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print("[work list]", *a, flush=True)
    sys.stdout.flush()


def _nat():
    import flash_attn  # noqa: F401
    from flash_attn import _native
    return _native


def _nan_like(t):
    return torch.full_like(t, float("nan"))


CASES = [
    # lengths, q heads, kv heads, head dim, causal, window
    ([2300, 700, 4100, 128, 3000, 2048, 513, 1, 3500, 2600], 16, 16, 128, True, (-1, -1)),     # ping-pong kernel, 2 heads per XCD
    ([2300, 0, 4100, 128, 3000, 0, 513, 2600], 32, 8, 128, True, (-1, -1)),                    # empty sequences; 4 grouped heads
    ([2500, 900, 3100, 2200, 640], 8, 1, 128, False, (-1, -1)),                                  # MQA cut into 8 parts, full mask
    ([2500, 900, 3100, 2200, 640], 16, 2, 128, False, (900, 100)),                               # GQA 2 kv heads x 4 parts, window
    ([600, 1500, 90, 1030, 777, 512, 64, 2000, 1200], 16, 16, 64, True, (-1, -1)),               # pipelined kernel, head dim 64
    ([600, 1500, 90, 1030, 777, 512, 64, 2000, 1200], 8, 8, 256, True, (-1, -1)),                # pair kernel, head dim 256
    ([600, 1500, 90, 1030, 777, 512], 16, 8, 192, True, (-1, -1)),                               # pair kernel, 192 columns
    ([2300, 700, 4100, 128, 3000, 2048, 513, 1], 16, 16, 96, True, (-1, -1)),                    # ping-pong kernel, 96 columns
    ([600, 1030, 90, 300, 2100], 12, 2, 128, True, (-1, -1)),                                    # 6 q heads per kv head: no list
    ([1, 2, 3], 8, 8, 128, True, (-1, -1)),                                                       # general kernel (short): no list
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "n%d_h%d_%d_d%d" % (len(c[0]), c[1], c[2], c[3]))
def test_work_list_equals_arithmetic_order(case):
    lens, h, hk, d, causal, window = case
    _say(case)
    nat = _nat()
    total, mx = sum(lens), max(lens)
    gen = torch.Generator().manual_seed(len(lens) * 1000 + d + h)
    q = torch.randn(total, h, d, generator=gen).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(total, hk, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32).to(DEV)

    def run(use_list):
        nat.WORK_LIST = use_list
        try:
            res = nat.varlen_fwd(q, k, v, _nan_like(q), cu, cu, mx, mx, 0.0, d ** -0.5, False, causal, window[0], window[1], False, None)
        finally:
            nat.WORK_LIST = True
        torch.cuda.synchronize()
        return res[0], res[5]

    out_a, lse_a = run(False)
    out_l, lse_l = run(True)
    assert not torch.isnan(out_l).any(), "rows no workgroup wrote"
    assert torch.equal(out_l, out_a)
    for i, n in enumerate(lens):
        assert torch.equal(lse_l[i][:, :n], lse_a[i][:, :n])


def test_work_list_many_sequences_and_replays():
    """300 sequences (the list builder ranks them quadratically in LDS), launched three times in a row on
    changing lengths with the same lent words: each launch rebuilds its list."""
    _say("many sequences")
    nat = _nat()
    h, d = 16, 128
    gen = torch.Generator().manual_seed(7)
    for rep in range(3):
        lens = torch.randint(0, 700, (300,), generator=gen).tolist()
        lens[rep] = 2600 + 100 * rep          # one long sequence picks the ping-pong kernel
        total, mx = sum(lens), max(lens)
        q, k, v = (torch.randn(total, h, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(3))
        cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32).to(DEV)
        outs = []
        for use_list in (False, True):
            nat.WORK_LIST = use_list
            try:
                res = nat.varlen_fwd(q, k, v, _nan_like(q), cu, cu, mx, mx, 0.0, d ** -0.5, False, True, -1, -1, False, None)
            finally:
                nat.WORK_LIST = True
            outs.append(res[0])
        torch.cuda.synchronize()
        assert not torch.isnan(outs[1]).any()
        assert torch.equal(outs[0], outs[1])


def test_work_list_words_reported_through_the_c_abi():
    import ctypes
    nat = _nat()
    p = nat.FaFwdParams()
    p.b, p.h, p.h_k, p.seqlen_q, p.d = 64, 16, 16, 4096, 128
    W = nat.WORK_COUNTER_WORDS
    assert nat.lib.fa_work_list_words(ctypes.byref(p)) == W       # dense batch: no list
    cu = torch.zeros(65, dtype=torch.int32, device=DEV)
    p.cu_seqlens_q = cu.data_ptr()
    # 64 sequences x 16 heads x 32 row blocks of 128 rows, two words each, + 8 counts + the ticket words
    assert nat.lib.fa_work_list_words(ctypes.byref(p)) == W + 8 + 2 * 64 * 16 * 32
    p.h, p.h_k = 12, 2                                             # 6 q heads per kv head cannot be cut into 8 / h_k parts
    assert nat.lib.fa_work_list_words(ctypes.byref(p)) == W
    p.h, p.h_k, p.b = 16, 16, 5000                                 # more sequences than the builder ranks
    assert nat.lib.fa_work_list_words(ctypes.byref(p)) == W


@pytest.mark.parametrize("lens,h,hk,d", [
    ([2300, 700, 4100, 128, 3000, 2048, 513, 1, 3500, 2600], 16, 16, 128),     # 256-row blocks, 2 heads of a sequence per XCD
    ([600, 1500, 0, 1030, 777, 512, 64, 2000], 32, 8, 64),                        # 128-row blocks, 4 grouped heads, an empty sequence
    ([2500, 900, 3100, 2200, 640], 8, 1, 128),                                     # MQA: 8 parts of one q head
])
def test_device_built_list_is_a_permutation_of_the_row_blocks(lens, h, hk, d):
    """Reads the list back from the lent words after a launch: every (sequence, q head, row block) that
    exists appears exactly once, on the XCD that owns its head, and nothing else appears."""
    _say("list contents", lens, h, hk, d)
    nat = _nat()
    total, mx = sum(lens), max(lens)
    gen = torch.Generator().manual_seed(11)
    q = torch.randn(total, h, d, generator=gen).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(total, hk, d, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(2))
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32).to(DEV)
    nat.varlen_fwd(q, k, v, None, cu, cu, mx, mx, 0.0, d ** -0.5, False, True, -1, -1, False, None)
    torch.cuda.synchronize()
    dev = q.device
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), nat._stream(dev))
    words = nat._COUNTERS[key].cpu().tolist()
    W = nat.WORK_COUNTER_WORDS
    assert not any(words[:W])                              # the ticket words stay zero
    counts, body = words[W:W + 8], words[W + 8:]
    block_m = 256 if d == 128 else 128                     # ping-pong kernel / pipelined kernel
    n_mb = [(n + block_m - 1) // block_m for n in lens]
    nmb_max = (mx + block_m - 1) // block_m
    per_xcd = len(lens) * h // 8 * nmb_max                 # slots per XCD list
    G = h // hk
    parts = 1 if hk > 2 or G % (8 // hk) else 8 // hk
    Gp = G // parts
    seen = set()
    for x in range(8):
        assert 0 <= counts[x] <= per_xcd
        for j in range(counts[x]):
            b, w = body[(x * per_xcd + j) * 2], body[(x * per_xcd + j) * 2 + 1]
            head, mb = (w >> 16) & 0xffff, w & 0xffff
            assert 0 <= b < len(lens) and head < h and mb < n_mb[b], (x, j, b, head, mb)
            hkp = (head // G) * parts + (head % G) // Gp       # kv head part the q head belongs to
            assert hkp % 8 == x, "q head %d on XCD %d" % (head, x)
            assert (b, head, mb) not in seen
            seen.add((b, head, mb))
    assert len(seen) == sum(n_mb) * h
