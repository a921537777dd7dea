"""CPU model of the running-maximum rule of the long-sequence forward kernels, checked numerically.

The kernels (csrc/fa_prefill_pp.h, csrc/fa_prefill_il.h) do not take a row maximum per key tile as the reference does
(softmax_rescale_o, csrc/flash_attn/src/flash_fwd_kernel.h:24-53).  Per tile of 64 keys and per query row they

  1. exponentiate the tile against the reference maximum m the row already has: p = 2^(s - m) (s in the log2 domain);
  2. accept the tile if its row sum is finite and at most 2^14;
  3. otherwise form the tile's exact maximum mx, move the reference to mx only if mx - m > 8, rescale the running sum
     and output by 2^(m_old - m_new), and exponentiate the tile again.

The argument for the two constants, restated here as executable checks on adversarial rows:
  * an accepted tile holds no probability above 2^14 (its sum bounds every term), which is finite in fp16 (max 65504)
    and exact enough in bf16; a redone tile holds none above 2^8 when the reference moved (then p <= 1) or stayed
    (mx - m <= 8);
  * the reference never exceeds the row's true running maximum (it is always a score the row has seen) and lags
    it by at most 14, so the row's largest probability is at least 1 and at most 2^14 in the kernel's units: the
    running sum neither underflows nor overflows in fp32 and the final o / l is exact up to fp32 rounding;
  * out and lse equal the plain softmax's up to fp32 rounding, whatever the order and size of the scores.
The model runs in float32 like the kernels and is compared with float64 softmax."""
import numpy as np
import pytest

TILE = 64


def lazy_softmax_row(s, v, tile=TILE):
    """One query row: s (n,) scores in the log2 domain, v (n, d).  Returns (out, lse2, stats) computed with the
    kernels' rule; -inf scores are masked keys."""
    s = s.astype(np.float32)
    m = np.float32(-np.inf)
    l = np.float32(0.0)
    o = np.zeros(v.shape[1], dtype=np.float32)
    pmax, lag_max, redo = 0.0, 0.0, 0
    true_max = -np.inf
    for t0 in range(0, len(s), tile):
        st = s[t0:t0 + tile]
        with np.errstate(invalid="ignore", over="ignore"):
            p = np.exp2(st - m).astype(np.float32)          # m = -inf: inf or nan, caught by the sum test
            tsum = np.float32(p.sum(dtype=np.float32))
        if not (tsum <= np.float32(16384.0)):
            redo += 1
            mx = np.float32(st.max())
            with np.errstate(invalid="ignore"):
                move = bool((mx - m) > np.float32(8.0))          # false for nan (-inf - -inf)
            m_new = mx if move else m
            with np.errstate(invalid="ignore"):
                corr = np.float32(np.exp2(m - m_new)) if move else np.float32(1.0)
            if np.isnan(corr):
                corr = np.float32(0.0)
            l = l * corr
            o = o * corr
            m = m_new
            ref = np.float32(0.0) if np.isneginf(m) else m
            p = np.exp2(st - ref).astype(np.float32)
            tsum = np.float32(p.sum(dtype=np.float32))
        l = np.float32(l + tsum)
        o = o + p @ v[t0:t0 + tile].astype(np.float32)
        if np.isfinite(st).any():
            true_max = max(true_max, float(st[np.isfinite(st)].max()))
        pmax = max(pmax, float(p.max()))
        if np.isfinite(m) and np.isfinite(true_max):
            assert m <= true_max + 1e-6                       # the reference is a score the row has seen
            lag_max = max(lag_max, true_max - float(m))
    if l == 0 or np.isnan(l):
        return np.zeros_like(o), np.inf, dict(pmax=pmax, lag=lag_max, redo=redo)
    return o / l, float(m) + float(np.log2(l)), dict(pmax=pmax, lag=lag_max, redo=redo)


def exact_row(s, v):
    s = s.astype(np.float64)
    fin = np.isfinite(s)
    if not fin.any():
        return np.zeros(v.shape[1]), np.inf
    mx = s[fin].max()
    p = np.where(fin, np.exp2(s - mx), 0.0)
    return (p @ v.astype(np.float64)) / p.sum(), mx + np.log2(p.sum())


def _rows(rng, n):
    base = rng.standard_normal(n) * 1.4427
    yield "gaussian", base
    yield "rising", base + np.linspace(-45, 45, n)
    yield "falling", base + np.linspace(45, -45, n)
    for name, j in (("spike_first", 3), ("spike_middle", n // 2 + 1), ("spike_last", n - 2)):
        s = base.copy()
        s[j] += 43.0
        yield name, s
    yield "steps_of_6", base + 6.0 * (np.arange(n) // TILE)               # a tile's sum stays under 2^14 one step out of two
    yield "steps_of_15", base + 15.0 * (np.arange(n) // TILE)             # every tile just outside
    yield "steps_of_7_9", base + np.cumsum(np.where(np.arange(n) % TILE == 0, 7.9, 0.0))   # lag builds up below 2^8
    yield "huge", base * 500.0
    s = base.copy()
    s[: 3 * TILE] = -np.inf
    yield "dead_start", s
    s = base.copy()
    s[2 * TILE: 5 * TILE] = -np.inf
    s[-TILE:] = -np.inf
    yield "dead_middle_and_end", s
    yield "all_masked", np.full(n, -np.inf)
    s = np.full(n, -np.inf)
    s[n - 1] = 5.0
    yield "one_key_last", s
    yield "constant_tile_at_bound", np.concatenate([np.zeros(TILE), np.full(TILE, 8.0), np.full(TILE, 14.0 - 6.0)])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_lazy_reference_rule_matches_exact_softmax(seed):
    rng = np.random.default_rng(seed)
    n, d = 16 * TILE, 8
    v = rng.standard_normal((n, d))
    for name, s in _rows(rng, n):
        vv = v[: len(s)]
        out, lse2, st = lazy_softmax_row(s, vv)
        ref, lse_ref = exact_row(s, vv)
        # no probability beyond what 16-bit storage and the fp32 sums take
        assert st["pmax"] <= 16384.0 * (1 + 1e-6), (name, st)
        assert st["lag"] <= 14.0 + 1e-3, (name, st)
        if np.isinf(lse_ref):
            assert np.isinf(lse2) and lse2 > 0 and not out.any(), name
            continue
        assert abs(lse2 - lse_ref) <= 1e-4 * max(1.0, abs(lse_ref)), (name, lse2, lse_ref)
        assert np.abs(out - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max()), (name, np.abs(out - ref).max())


def test_branch_fires_where_the_argument_says():
    """Gaussian rows redo only their first tile; a ramp of 15 per tile redoes every tile; a ramp of 6 per tile is
    accepted while the tile's sum stays under 2^14 and redone, with the reference moved, when it does not."""
    rng = np.random.default_rng(5)
    n, d = 16 * TILE, 4
    v = rng.standard_normal((n, d))
    rows = dict(_rows(rng, n))
    assert lazy_softmax_row(rows["gaussian"], v)[2]["redo"] == 1
    assert lazy_softmax_row(rows["steps_of_15"], v)[2]["redo"] == 16
    r6 = lazy_softmax_row(rows["steps_of_6"], v)[2]
    assert 1 < r6["redo"] < 16 and r6["lag"] <= 14.0 + 1e-3
    assert lazy_softmax_row(rows["dead_start"], v)[2]["redo"] >= 4           # three dead tiles, then the first live one


def test_fp16_storage_of_accepted_probabilities():
    """the largest accepted probability, 2^14, is exact and finite in fp16 (bf16 has fp32's range)"""
    assert float(np.float32(16384.0).astype(np.float16)) == 16384.0
    assert np.isfinite(np.float32(16384.0 * 1.999).astype(np.float16))
