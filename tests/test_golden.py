"""The committed fixtures of tests/golden/ (inputs with the oracle's outputs and gradients, written by
tests/golden/make_golden.py): on the CPU the oracle must still reproduce them exactly; on the GPU the HIP
kernels are compared with the stored values under the usual acceptance rules."""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import attention_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

DATA = np.load(os.path.join(HERE, "golden", "attention_cases.npz"))


def _t(name, dtype=torch.float32):
    return torch.from_numpy(DATA[name]).to(dtype)


def test_oracle_reproduces_fixtures():
    fresh = make_golden.build()
    assert sorted(fresh) == sorted(DATA.files)
    for key in DATA.files:
        assert np.array_equal(fresh[key], DATA[key]), key


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(make_golden.CASES))
def test_kernels_match_fixtures(name):
    import flash_attn
    b, sq, sk, h, hk, d, dtype, causal, window = make_golden.CASES[name]
    print("golden", name, flush=True)
    q, k, v, dout = (_t(name + "." + n, dtype).cuda() for n in ("q", "k", "v", "dout"))
    q.requires_grad_(); k.requires_grad_(); v.requires_grad_()
    out, lse, _ = flash_attn.flash_attn_func(q, k, v, causal=causal, window_size=window, return_attn_probs=True)
    ok, err, bound = orc.tolerance_ok(out.detach().cpu(), _t(name + ".out"), _t(name + ".out_lowprec"), 2.0, 1e-5)
    assert ok, (err, bound)
    assert orc.lse_ok(lse.cpu(), _t(name + ".lse"))[0]
    grads = torch.autograd.grad(out, (q, k, v), dout)
    for gname, got in zip(("dq", "dk", "dv"), grads):
        ref, low = _t(name + "." + gname), _t(name + "." + gname + "_lowprec")
        err = (got.float().cpu() - ref).abs().max().item()
        assert err <= 2 * (low - ref).abs().max().item() + 1e-5, (gname, err)


@pytest.mark.gpu
@pytest.mark.parametrize("interleaved", [False, True])
def test_rotary_matches_fixture(interleaved):
    from flash_attn.layers.rotary import apply_rotary_emb
    print("golden rotary", interleaved, flush=True)
    x = _t("rotary.x", torch.bfloat16).cuda()
    cos, sin = _t("rotary.cos", torch.bfloat16).cuda(), _t("rotary.sin", torch.bfloat16).cuda()
    offsets = torch.from_numpy(DATA["rotary.offsets"]).cuda()
    got = apply_rotary_emb(x, cos, sin, interleaved=interleaved, seqlen_offsets=offsets).float().cpu()
    want = _t("rotary.out_interleaved" if interleaved else "rotary.out_halves")
    # one bf16 unit in the last place where a fused multiply-add moves a rounding tie
    assert torch.allclose(got, want, rtol=2 ** -7, atol=1e-6)
    assert (got != want).float().mean().item() < 0.02
