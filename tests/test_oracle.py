"""Pins the CPU oracle (oracle/awq_ref.py, oracle/awq_ref.c) with checks that do not retype
its formulas: hand-derived known answers, algebraic invariants, exact-rational brute force,
library routines, and agreement between the two independent derivations."""
import bisect
import json
import os
from fractions import Fraction

import numpy as np
import pytest

from oracle import awq_ref, cref

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ------------------------------------------------------------------ nibble order

def test_pack_known_answers():
    kat = json.load(open(os.path.join(GOLDEN, "nibble_kat.json")))
    for case in kat["pack"]:
        got = awq_ref.pack_awq(np.array([case["logical"]]))[0, 0]
        assert (int(got) & 0xFFFFFFFF) == int(case["word"], 16)
        assert int(got) == case["int32"]
    for case in kat["unpack"]:
        w = np.array([[int(case["word"], 16)]], dtype=np.uint32).view(np.int32)
        assert awq_ref.unpack_awq(w)[0].tolist() == case["logical"]
        assert cref.unpack(w)[0].tolist() == case["logical"]


def test_orders_are_inverse():
    P, R = awq_ref.AWQ_PACK_ORDER, awq_ref.AWQ_UNPACK_ORDER
    assert [R[P[i]] for i in range(8)] == list(range(8))
    assert [P[R[j]] for j in range(8)] == list(range(8))
    assert sorted(P) == list(range(8))


def test_single_nibble_positions():
    # logical column j alone set to 0xF must light exactly nibble R[j]; derived from
    # "nibble i stores logical column P[i]", not from the oracle's shift table
    P = [0, 2, 4, 6, 1, 3, 5, 7]
    for j in range(8):
        v = np.zeros((1, 8), np.int64)
        v[0, j] = 0xF
        word = int(awq_ref.pack_awq(v)[0, 0]) & 0xFFFFFFFF
        nib = P.index(j)
        assert word == 0xF << (4 * nib)


def test_roundtrip_and_sign_bit():
    rng = np.random.default_rng(1)
    v = rng.integers(0, 16, size=(37, 64))
    packed = awq_ref.pack_awq(v)
    assert packed.dtype == np.int32
    assert np.array_equal(awq_ref.unpack_awq(packed), v)
    assert np.array_equal(cref.unpack(packed), v)
    # column 7 lives in bits 28..31: words >= 2^31 are negative int32, still unpack to 8..15
    v = np.zeros((1, 8), np.int64)
    v[0, 7] = 15
    p = awq_ref.pack_awq(v)
    assert p[0, 0] < 0
    assert awq_ref.unpack_awq(p)[0, 7] == 15 and cref.unpack(p)[0, 7] == 15


# ------------------------------------------------------------------ fp16 conversion of the C oracle

def test_c_half_conversions_match_numpy():
    L = cref.lib()
    halves = np.arange(65536, dtype=np.uint16)
    as_f = halves.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        f = L.awqref_h2f(h)
        if np.isnan(as_f[h]):
            assert np.isnan(f)
        else:
            assert f == as_f[h]
    rng = np.random.default_rng(2)
    # normal range, subnormal range, overflow edge, ties
    samples = np.concatenate([
        rng.normal(0, 1, 4000).astype(np.float32),
        (rng.random(4000) * 1.3e-4).astype(np.float32),
        (rng.random(2000) * 1.2e-7).astype(np.float32),
        np.array([65504.0, 65519.9, 65520.0, 70000.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 0.0, -0.0], np.float32),
    ])
    samples = np.concatenate([samples, -samples])
    with np.errstate(over="ignore"):
        want = samples.astype(np.float16).view(np.uint16)
    for f, w in zip(samples.tolist(), want.tolist()):
        assert L.awqref_f2h(f) == w, (f, w)


# ------------------------------------------------------------------ dequantize

def _all_scales_in_range():
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    with np.errstate(invalid="ignore"):
        m = (h >= np.float16(0.001)) & (h <= np.float16(0.02))
    return h[m]


def _dequant_grid(scales_1d):
    """qweight/qzeros/scales such that every (w, z) pair meets every scale: K = 16 rows
    (w = row), one group; column block per z."""
    S = scales_1d.size
    N = 16 * S
    N8 = (N + 7) // 8 * 8
    w = np.repeat(np.arange(16)[:, None], N8, axis=1)
    z = np.zeros((1, N8), np.int64)
    s = np.ones((1, N8), np.float16)
    for zz in range(16):
        z[0, zz * S:(zz + 1) * S] = zz
        s[0, zz * S:(zz + 1) * S] = scales_1d
    return awq_ref.pack_awq(w), s, awq_ref.pack_awq(z), w, z, s


def test_dequant_exhaustive_float64_route():
    """Every (w, z) pair x every fp16 scale in [0.001, 0.02]: the exact product fits a
    float64, and numpy's float64 -> float16 cast is a single correct rounding."""
    sc = _all_scales_in_range()
    assert 4000 < sc.size < 5000
    qw, s, qz, w, z, _ = _dequant_grid(sc)
    want = ((w - z).astype(np.float64) * s.astype(np.float64)).astype(np.float16)
    got_np = awq_ref.dequantize(qw, s, qz, 16)
    got_c = cref.dequantize(qw, s, qz, 16)
    assert np.array_equal(got_np.view(np.uint16), want.view(np.uint16))
    assert np.array_equal(got_c.view(np.uint16), want.view(np.uint16))


def test_dequant_exact_rational_sample():
    """Exact rational product, nearest fp16 by search over the sorted table of all finite
    fp16 values, ties to even mantissa; shares no code with either oracle."""
    table = np.arange(0x7C00, dtype=np.uint16)             # non-negative finite halves
    vals = [Fraction(float(x)) for x in table.view(np.float16).astype(np.float64)]

    def nearest(fr):
        sign = fr < 0
        a = -fr if sign else fr
        i = bisect.bisect_left(vals, a)
        if i == len(vals):
            cand = len(vals) - 1
        elif i == 0:
            cand = 0
        else:
            lo, hi = vals[i - 1], vals[i]
            if a - lo < hi - a:
                cand = i - 1
            elif a - lo > hi - a:
                cand = i
            else:
                cand = i - 1 if (i - 1) % 2 == 0 else i
        return int(table[cand]) | (0x8000 if sign and cand != 0 else 0) | (0x8000 if sign and cand == 0 else 0)

    rng = np.random.default_rng(3)
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = allh[np.isfinite(allh) & (np.abs(allh.astype(np.float32)) < 4000)]
    sc = rng.choice(finite, size=300)
    sc[:6] = np.array([6.1e-5, 5.96e-8, 1e-7, 0.001, 0.02, 3e-5], np.float16)   # subnormal-adjacent too
    qw, s, qz, w, z, _ = _dequant_grid(sc)
    got_np = awq_ref.dequantize(qw, s, qz, 16).view(np.uint16)
    got_c = cref.dequantize(qw, s, qz, 16).view(np.uint16)
    assert np.array_equal(got_np, got_c)
    for r in range(16):
        for c in rng.choice(w.shape[1], size=120, replace=False):
            want = nearest(Fraction(int(w[r, c] - z[0, c])) * Fraction(float(s[0, c])))
            got = int(got_np[r, c])
            if (got & 0x7FFF) == 0 and (want & 0x7FFF) == 0:
                continue   # +0 / -0: sign of zero follows IEEE multiply, checked below
            assert got == want, (r, c, w[r, c], z[0, c], float(s[0, c]))


def test_dequant_special_cases_and_group_boundary():
    rng = np.random.default_rng(4)
    K, N, G = 256, 32, 128
    w = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // G, N))
    s = (rng.random((K // G, N)) * 0.019 + 0.001).astype(np.float16)
    # w == z on row 5 -> exactly +0.0 for positive scales
    w[5] = z[0]
    W = awq_ref.dequantize(awq_ref.pack_awq(w), s, awq_ref.pack_awq(z), G)
    assert np.all(W[5].view(np.uint16) == 0)
    # rows 127 / 128 straddle the group boundary: each must use its own (z, s)
    for k, g in ((127, 0), (128, 1)):
        want = ((w[k] - z[g]).astype(np.float64) * s[g].astype(np.float64)).astype(np.float16)
        assert np.array_equal(W[k].view(np.uint16), want.view(np.uint16))
    # linear in (w - z): doubling the integer difference doubles the value when no rounding
    assert np.array_equal(cref.dequantize(awq_ref.pack_awq(w), s, awq_ref.pack_awq(z), G).view(np.uint16),
                          W.view(np.uint16))
    # group = -1 means one group over all K
    s1, z1 = s[:1], z[:1]
    Wall = awq_ref.dequantize(awq_ref.pack_awq(w), s1, awq_ref.pack_awq(z1), -1)
    want = ((w - z1).astype(np.float64) * s1.astype(np.float64)).astype(np.float16)
    assert np.array_equal(Wall.view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------ gemm

def _case(M, K, N, G, seed):
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // G, N))
    s = (rng.random((K // G, N)) * 0.019 + 0.001).astype(np.float16)
    x = rng.normal(0, 1, (M, K)).astype(np.float16)
    return x, awq_ref.pack_awq(w), s, awq_ref.pack_awq(z), w, z


def test_gemm_one_hot_and_zero():
    x, qw, s, qz, w, z = _case(4, 256, 64, 128, 5)
    W = awq_ref.dequantize(qw, s, qz, 128)
    for k in (0, 127, 128, 255):
        e = np.zeros((1, 256), np.float16)
        e[0, k] = 1
        assert np.array_equal(awq_ref.gemm(e, qw, s, qz, 128).view(np.uint16)[0], W[k].view(np.uint16))
        assert np.array_equal(cref.gemm(e, qw, s, qz, 128)[0].view(np.uint16)[0], W[k].view(np.uint16))
    qw0 = awq_ref.pack_awq(np.repeat(z, 128, axis=0))
    assert not awq_ref.gemm(x, qw0, s, qz, 128).any()


def test_gemm_against_library_float64_and_c():
    x, qw, s, qz, w, z = _case(16, 512, 256, 128, 6)
    # library routine on independently dequantised weights (float64 everywhere)
    Wd = ((w - np.repeat(z, 128, axis=0)).astype(np.float64)
          * np.repeat(s.astype(np.float64), 128, axis=0)).astype(np.float16).astype(np.float64)
    ref = x.astype(np.float64) @ Wd
    y32 = awq_ref.gemm(x, qw, s, qz, 128)
    yc, ywide = cref.gemm(x, qw, s, qz, 128)
    assert np.allclose(ywide, ref, rtol=1e-12, atol=1e-12)
    assert awq_ref.rel_frobenius(y32, ref) < 4e-4          # one fp16 rounding of the output
    assert awq_ref.rel_frobenius(yc, ref) < 4e-4
    assert np.allclose(awq_ref.gemm_wide(x, qw, s, qz, 128), ref, rtol=1e-12, atol=1e-12)
    # linearity in x
    y2 = awq_ref.gemm_wide((2 * x.astype(np.float32)).astype(np.float16), qw, s, qz, 128)
    assert np.allclose(y2, 2 * ref, rtol=1e-12, atol=1e-12)


def test_golden_fixture_matches_oracle():
    fx = np.load(os.path.join(GOLDEN, "awq_small.npz"))
    W = awq_ref.dequantize(fx["qweight"], fx["scales"], fx["qzeros"], int(fx["group"]))
    assert np.array_equal(W.view(np.uint16), fx["w_dequant_bits"])
    assert np.array_equal(cref.dequantize(fx["qweight"], fx["scales"], fx["qzeros"], int(fx["group"]))
                          .view(np.uint16), fx["w_dequant_bits"])
    y = awq_ref.gemm_wide(fx["x"], fx["qweight"], fx["scales"], fx["qzeros"], int(fx["group"]))
    assert np.allclose(y, fx["y_f64"], rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ MoE

@pytest.mark.parametrize("T,E,topk,tile", [(1, 8, 2, 16), (7, 4, 2, 4), (64, 128, 8, 16), (33, 16, 4, 16)])
def test_moe_align_invariants(T, E, topk, tile):
    rng = np.random.default_rng(T * 131 + E)
    ids = np.stack([rng.choice(E, size=topk, replace=False) for _ in range(T)]).astype(np.int32)
    n = T * topk
    for impl in (awq_ref.moe_align, cref.moe_align):
        sorted_ids, expert_ids, npp = impl(ids, E, tile)
        assert npp == sorted_ids.size and npp % tile == 0
        real = sorted_ids[sorted_ids < n]
        assert sorted(real.tolist()) == list(range(n))                      # a permutation
        assert np.all(sorted_ids[sorted_ids >= n] == n)                     # pads are the sentinel
        counts = np.bincount(ids.reshape(-1), minlength=E)
        assert npp == int(sum(-(-c // tile) * tile for c in counts))
        assert expert_ids.size == npp // tile
        flat = ids.reshape(-1)
        for b in range(npp // tile):
            blk = sorted_ids[b * tile:(b + 1) * tile]
            realb = blk[blk < n]
            assert realb.size > 0
            assert np.all(flat[realb] == expert_ids[b])
            assert np.all(np.diff(realb) > 0)                               # stable inside a run
            assert np.all(blk[:realb.size] < n)                             # pads at the back
        assert np.all(np.diff(expert_ids) >= 0)
    a, b = awq_ref.moe_align(ids, E, tile), cref.moe_align(ids, E, tile)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]


def test_topk_softmax_against_torch():
    import torch
    g = torch.Generator().manual_seed(7)
    logits = torch.randn((64, 128), generator=g)
    ids, w = awq_ref.topk_softmax(logits.numpy(), 8, True)
    p = torch.softmax(logits.double(), dim=-1)
    tw, ti = torch.topk(p, 8, dim=-1)
    tw = tw / tw.sum(-1, keepdim=True)
    assert np.array_equal(ids, ti.numpy().astype(np.int32))
    assert np.allclose(w, tw.numpy(), rtol=1e-6)
    ids2, w2 = awq_ref.topk_softmax(logits.numpy(), 8, False)
    assert np.allclose(w2, torch.topk(p, 8, dim=-1)[0].numpy(), rtol=1e-6)
    # ties resolve to the lowest expert id
    tie = np.zeros((1, 8), np.float32)
    assert awq_ref.topk_softmax(tie, 3)[0].tolist() == [[0, 1, 2]]


def test_moe_forward_against_grouped_formulation():
    """The per-token loop must equal the expert-grouped evaluation (gather rows per expert,
    one matmul per expert), which is how the device computes it."""
    rng = np.random.default_rng(8)
    T, H, E, topk, I, G = 5, 256, 4, 2, 128, 128

    def stack(K, N):
        w = rng.integers(0, 16, (E, K, N))
        z = rng.integers(0, 16, (E, K // G, N))
        s = (rng.random((E, K // G, N)) * 0.019 + 0.001).astype(np.float16)
        return awq_ref.pack_awq(w), s, awq_ref.pack_awq(z)

    w13, w2 = stack(H, 2 * I), stack(I, H)
    x = rng.normal(0, 1, (T, H)).astype(np.float16)
    logits = rng.normal(0, 1, (T, E)).astype(np.float32)
    ids, tw = awq_ref.topk_softmax(logits, topk)
    got = awq_ref.moe_forward(x, w13, w2, ids, tw, G).astype(np.float64)
    want = np.zeros((T, H))
    for e in range(E):
        W13 = awq_ref.dequantize(w13[0][e], w13[1][e], w13[2][e], G).astype(np.float64)
        W2 = awq_ref.dequantize(w2[0][e], w2[1][e], w2[2][e], G).astype(np.float64)
        for t, slot in zip(*np.nonzero(ids == e)):
            h = x[t].astype(np.float64) @ W13
            a = h[:I] / (1 + np.exp(-h[:I])) * h[I:]
            want[t] += (a @ W2) * tw[t, slot]
    assert awq_ref.rel_frobenius(got, want) < 2e-3


def test_topk_sigmoid_matches_torch():
    import torch
    """sigmoid scoring with a correction bias: ids from torch.topk of score + bias, weights the
    plain scores (random floats: no ties), renormalised and scaled."""
    g = torch.Generator().manual_seed(11)
    logits = torch.randn((9, 40), generator=g)
    bias = torch.randn((40,), generator=g) * 0.1
    score = torch.sigmoid(logits.double())
    choice = score.float() + bias
    ids_t = torch.topk(choice, 5, dim=-1).indices
    w_t = score.gather(1, ids_t)
    w_t = w_t / w_t.sum(dim=-1, keepdim=True) * 2.5
    ids, w = awq_ref.topk_sigmoid(logits.numpy(), 5, True, bias.numpy(), 2.5)
    assert np.array_equal(ids, ids_t.numpy().astype(np.int32))
    assert np.allclose(w, w_t.numpy(), rtol=1e-6)
    ids2, w2 = awq_ref.topk_sigmoid(logits.numpy(), 5, False)
    assert np.array_equal(ids2, torch.topk(score, 5, dim=-1).indices.numpy().astype(np.int32))
    assert np.allclose(w2, torch.topk(score, 5, dim=-1).values.numpy(), rtol=1e-6)


def test_cpu_baseline_functions_against_the_pinned_oracle():
    """The PyTorch functions that the benchmark times as the CPU baseline (and uses to check GPU
    results at benchmark sizes): their dequantised weights carry the oracle's bits, and their
    products equal the oracle's fp32-accumulated ones up to the summation order of the two
    libraries (one fp16 ulp on a few elements, far inside 2e-3 of the float64 product)."""
    import torch
    import server_benchmark_amd as sba
    c = sba.workloads.config0()                    # M = 16, K = N = 4096, group 128, seed 0
    x, qw, s, qz = (t.numpy() for t in (c.x, c.qweight, c.scales, c.qzeros))
    Wt = awq_ref.cpu_dequantize_torch(c.qweight, c.scales, c.qzeros, 128).numpy()
    assert np.array_equal(Wt.view(np.uint16), awq_ref.dequantize(qw, s, qz, 128).view(np.uint16))
    yt = awq_ref.cpu_linear_torch(c.x, c.qweight, c.scales, c.qzeros, 128).numpy()
    yn = awq_ref.gemm(x, qw, s, qz, 128, acc=np.float32)
    # one fp16 ulp apart at most, plus the fp32 summation-order noise where the sum cancels
    d = np.abs(yt.astype(np.float64) - yn.astype(np.float64))
    assert np.all(d <= 2.0 ** -10 * np.abs(yn.astype(np.float64)) + 1e-4)
    assert (yt.view(np.uint16) == yn.view(np.uint16)).mean() >= 0.99
    assert awq_ref.rel_frobenius(yt, awq_ref.gemm_wide(x, qw, s, qz, 128)) <= 4e-4
    # group = -1 (one group over K) and the MoE form against the per-token brute force
    m = sba.workloads.make_moe_case(5, 256, 8, 2, 128, 128, seed=9)
    ids, tw = awq_ref.topk_softmax(m.logits.numpy(), 2, True)
    want = awq_ref.moe_forward(m.x.numpy(), tuple(a.numpy() for a in m.w13), tuple(a.numpy() for a in m.w2),
                               ids, tw, 128)
    got = awq_ref.cpu_moe_torch(m.x, m.w13, m.w2, torch.from_numpy(ids), torch.from_numpy(tw), 128).numpy()
    assert awq_ref.rel_frobenius(got, want) <= 1e-3
