"""GPU parity: the HIP kernels, called through the C ABI (ctypes), against the CPU oracle on
the same seeded inputs.  Integer / dequant results must be bit-exact; GEMM outputs must be
within a relative Frobenius error of 2e-3 of the float64 product of the fp16 inputs and the
pinned fp16 weights (TOL below), max-abs error printed."""
import os

import numpy as np
import pytest
import torch

from oracle import awq_ref

pytestmark = pytest.mark.gpu
TOL = 2e-3
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _np_case(M, K, N, G, seed):
    rng = np.random.default_rng(seed)
    g = K if G <= 0 else G
    w = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // g, N))
    s = (rng.random((K // g, N)) * 0.019 + 0.001).astype(np.float16)
    x = rng.normal(0, 1, (M, K)).astype(np.float16)
    return x, awq_ref.pack_awq(w), s, awq_ref.pack_awq(z)


def _dev(dev, *arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in arrs]


def _check_gemm(sba, dev, x, qw, s, qz, G, split_k=0, tag="", variant=None):
    ref = awq_ref.gemm_wide(x, qw, s, qz, G)
    xd, qwd, sd, qzd = _dev(dev, x, qw, s, qz)
    y = sba.awq_gemm(xd, qwd, sd, qzd, force_split_k=split_k, _dev_variant=variant)
    torch.cuda.synchronize()
    yh = y.cpu().numpy()
    err = awq_ref.rel_frobenius(yh, ref)
    maxabs = float(np.max(np.abs(yh.astype(np.float64) - ref)))
    print(f"[gemm {tag} M={x.shape[0]} K={x.shape[1]} N={qw.shape[1] * 8} G={G} split={split_k}] "
          f"rel_fro={err:.2e} max_abs={maxabs:.3e}", flush=True)
    assert np.isfinite(yh).all()
    assert err <= TOL
    return yh


# ------------------------------------------------------------------ dequantize (bit-exact)

@pytest.mark.parametrize("K,N,G", [(256, 64, 128), (4096, 4096, 128), (128, 8, 32), (96, 40, 24),
                                   (64, 2056, 64), (384, 128, -1), (30, 16, 3), (512, 264, 256)])
def test_dequantize_bit_exact(sba, gpu, K, N, G):
    _, qw, s, qz = _np_case(1, K, N, G, seed=K + N)
    want = awq_ref.dequantize(qw, s, qz, G)
    qwd, sd, qzd = _dev(gpu, qw, s, qz)
    got = sba.awq_dequantize(qwd, sd, qzd, 0, 0, 0).cpu().numpy()
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_dequantize_exhaustive_and_fixture(sba, gpu):
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    with np.errstate(invalid="ignore"):
        finite = h[np.isfinite(h)]
    # every finite fp16 scale (subnormal results included) x every (w, z) pair
    S = finite.size
    N = 16 * S
    N8 = (N + 7) // 8 * 8
    w = np.repeat(np.arange(16)[:, None], N8, axis=1)
    z = np.zeros((1, N8), np.int64)
    s = np.ones((1, N8), np.float16)
    for zz in range(16):
        z[0, zz * S:(zz + 1) * S] = zz
        s[0, zz * S:(zz + 1) * S] = finite
    qw, qz = awq_ref.pack_awq(w), awq_ref.pack_awq(z)
    with np.errstate(over="ignore"):
        want = ((w - z).astype(np.float64) * s.astype(np.float64)).astype(np.float16)
    got = sba.awq_dequantize(*_dev(gpu, qw, s, qz), 0, 0, 0).cpu().numpy()
    gb, wb = got.view(np.uint16), want.view(np.uint16)
    same = (gb == wb) | (((gb | wb) & 0x7FFF) == 0)     # +0 / -0 both fine
    assert same.all(), np.argwhere(~same)[:5]

    fx = np.load(os.path.join(GOLDEN, "awq_small.npz"))
    got = sba.awq_dequantize(*_dev(gpu, fx["qweight"], fx["scales"], fx["qzeros"]), 0, 0, 0).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), fx["w_dequant_bits"])


# ------------------------------------------------------------------ decode GEMM (M <= 16)

@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("M", [1, 4, 8, 16])
def test_gemm_decode_small(sba, gpu, M, variant):
    x, qw, s, qz = _np_case(M, 1024, 512, 128, seed=10 + M)
    for split in (0, 1, 2, 3, 8):
        _check_gemm(sba, gpu, x, qw, s, qz, 128, split, tag=f"v{variant}", variant=variant)


@pytest.mark.parametrize("K,N,G", [(256, 128, 32), (256, 264, 64), (512, 136, 256), (384, 8, -1),
                                   (128, 2048, 128), (640, 1000, 128)])
def test_gemm_decode_groups_and_ragged_n(sba, gpu, K, N, G):
    x, qw, s, qz = _np_case(5, K, N, G, seed=K * 3 + N)
    g = K if G <= 0 else G
    for split in (0, 1, 2):
        _check_gemm(sba, gpu, x, qw, s, qz, g, split)


@pytest.mark.parametrize("K,N,split,M", [(640, 256, 1, 16), (1152, 512, 1, 3), (1152, 512, 2, 16),
                                         (4736, 256, 8, 1), (4736, 264, 8, 16), (29568, 256, 8, 7)])
def test_gemm_decode_left_over_chunks_step_by_step(sba, gpu, K, N, split, M):
    """Chunk counts that leave L chunks over after each of the 4 x split waves got the same
    number, with 4 L <= waves: the left-over chunks are taken one 32-row step per wave (all
    waves, some of them, or - N = 264 - in the one-word-per-lane form that never does).  Checked
    against the oracle, against the whole-chunk form (development variant bit 1 << 23) within tolerance, and
    exactly with one-hot activations that sit inside the left-over chunks."""
    x, qw, s, qz = _np_case(M, K, N, 128, seed=K + N + split)
    y = _check_gemm(sba, gpu, x, qw, s, qz, 128, split, tag="tail steps")
    y_whole = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), force_split_k=split, _dev_variant=1 << 23).cpu().numpy()
    assert awq_ref.rel_frobenius(y, y_whole.astype(np.float64)) <= 1e-3
    W = awq_ref.dequantize(qw, s, qz, 128)
    nchunks, parts = K // 128, 4 * split
    first_left = (nchunks // parts) * parts * 128          # first row of the left-over chunks
    ks = [0, first_left - 1, first_left, first_left + 31, first_left + 32, first_left + 100, K - 33, K - 1]
    xo = np.zeros((len(ks), K), np.float16)
    for m, k in enumerate(ks):
        xo[m, k] = 1
    yo = sba.awq_gemm(*_dev(gpu, xo, qw, s, qz), force_split_k=split).cpu().numpy()
    for m, k in enumerate(ks):
        assert np.array_equal(yo[m].view(np.uint16), W[k].view(np.uint16)), (m, k)


@pytest.mark.parametrize("M", [17, 24, 32, 33, 48, 64])
def test_gemm_mid_m_skinny_passes(sba, gpu, M):
    """17 <= M <= 64 runs the skinny kernel in passes of up to 32 rows (two row blocks share
    every unpacked weight)."""
    x, qw, s, qz = _np_case(M, 1024, 512, 128, seed=200 + M)
    for split in (0, 1, 4):
        _check_gemm(sba, gpu, x, qw, s, qz, 128, split, tag="mid-M")
    x, qw, s, qz = _np_case(M, 512, 264, 64, seed=300 + M)      # ragged N, G = 64
    _check_gemm(sba, gpu, x, qw, s, qz, 64, 0, tag="mid-M")


@pytest.mark.parametrize("M,K,N,G,split", [(17, 4096, 264, 128, 1), (32, 3072, 2048, 64, 1), (24, 12288, 512, 128, 0),
                                           (32, 8192, 256, 1024, 2)])
def test_gemm_32_row_pass_with_lds_weight_ring(sba, gpu, M, K, N, G, split):
    """17 .. 32 rows over long wave ranges keep the weight ring in LDS; the register-ring form
    (development variant bit 4096) must give the same bits."""
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + K)
    y = _check_gemm(sba, gpu, x, qw, s, qz, G, split, tag="32-row lds ring")
    y_reg = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), force_split_k=split, _dev_variant=4096).cpu().numpy()
    assert np.array_equal(y.view(np.uint16), y_reg.view(np.uint16))


@pytest.mark.parametrize("M", [32, 33, 48, 64])
def test_gemm_wide_layer_mid_m(sba, gpu, M):
    """More than 128 column tiles: 32 rows run as one skinny pass, 33 .. 64 rows on the 64-row
    MFMA tile, whose tiles alone exceed one round of workgroups here."""
    x, qw, s, qz = _np_case(M, 256, 32768 + 512, 128, seed=M)
    _check_gemm(sba, gpu, x, qw, s, qz, 128, 0, tag="wide-mid-M")


def test_gemm_one_hot_is_exact_and_zero_weights(sba, gpu):
    K, N, G = 512, 256, 128
    _, qw, s, qz = _np_case(1, K, N, G, seed=77)
    W = awq_ref.dequantize(qw, s, qz, G)
    rows = [0, 1, 127, 128, 300, 511, 37, 64, 200, 255, 256, 383, 384, 385, 450, 9]
    x = np.zeros((16, K), np.float16)
    for m, k in enumerate(rows):
        x[m, k] = 1
    for split in (1, 4):
        y = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), force_split_k=split).cpu().numpy()
        for m, k in enumerate(rows):
            assert np.array_equal(y[m].view(np.uint16), W[k].view(np.uint16)), (split, m, k)
    # w == z everywhere: the reference gives exact zeros.  The skinny kernel sums x * w on the
    # matrix core and subtracts z * sum(x) through a separate MFMA, so what is left is fp32
    # cancellation noise: bound it by 2^-18 of the magnitude a full-scale weight would give
    # (|x|_1 * 15 * s_max), four orders of magnitude inside the 2e-3 tolerance.
    zfull = np.repeat(awq_ref.unpack_awq(qz), G, axis=0)
    xr = np.random.default_rng(0).normal(0, 1, (16, K)).astype(np.float16)
    y = sba.awq_gemm(*_dev(gpu, xr, awq_ref.pack_awq(zfull), s, qz), 0).cpu().numpy()
    bound = np.abs(xr.astype(np.float64)).sum(axis=1, keepdims=True) * 15 * float(s.max()) * 2.0 ** -18
    print(f"[w == z] max |y| = {np.abs(y).max():.3e}, bound {bound.min():.3e}", flush=True)
    assert np.all(np.abs(y.astype(np.float64)) <= bound)
    # the MFMA path (M > 64) dequantises to exact fp16 zeros first: exact zeros there
    xl = np.random.default_rng(1).normal(0, 1, (80, K)).astype(np.float16)
    assert not sba.awq_gemm(*_dev(gpu, xl, awq_ref.pack_awq(zfull), s, qz), 0).cpu().numpy().any()


@pytest.mark.parametrize("K,N,G,M", [(4096, 256, -1, 5), (4096, 512, 128, 16), (1024, 264, 1024, 3), (2048, 256, 256, 32)])
def test_gemm_decode_large_mean_and_outlier_activations(sba, gpu, K, N, G, M):
    """The skinny kernel takes the zero point out through a lane's running sum of x fed to the
    matrix core as fp16 pieces: activations with a large mean (sums of tens of thousands per lane
    and group, more with one group over all of K) or massive outliers must neither overflow that
    sum nor cost accuracy.  Checked against the float64 product with a max-abs bound next to the
    relative Frobenius one."""
    rng = np.random.default_rng(K + N + M)
    g = K if G <= 0 else G
    w = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // g, N))
    s = (rng.random((K // g, N)) * 0.019 + 0.001).astype(np.float16)
    qw, qz = awq_ref.pack_awq(w), awq_ref.pack_awq(z)
    cases = {
        "mean 100": rng.normal(100.0, 1.0, (M, K)),
        "mean -3000": rng.normal(-3000.0, 10.0, (M, K)),
        "outliers": rng.normal(0.0, 1.0, (M, K)),
    }
    cases["outliers"][:, rng.integers(0, K, 6)] = 30000.0
    cases["outliers"][:, rng.integers(0, K, 6)] = -28000.0
    for name, x in cases.items():
        x = x.astype(np.float16)
        ref = awq_ref.gemm_wide(x, qw, s, qz, g)
        if np.abs(ref).max() >= 60000:      # keep the true result inside fp16
            x = (x.astype(np.float32) * (30000.0 / np.abs(ref).max())).astype(np.float16)
            ref = awq_ref.gemm_wide(x, qw, s, qz, g)
        y = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0).cpu().numpy().astype(np.float64)
        assert np.isfinite(y).all(), name
        err = awq_ref.rel_frobenius(y, ref)
        maxabs = float(np.abs(y - ref).max())
        scale = float(np.abs(ref).max())
        print(f"[gemm {name} M={M} K={K} N={N} G={g}] rel_fro={err:.2e} max_abs={maxabs:.3e} of {scale:.3e}", flush=True)
        assert err <= TOL, name
        assert maxabs <= 2e-3 * scale, name


def test_gemm_config0(sba, gpu):
    c = sba.workloads.config0()
    x, qw, s, qz = (t.numpy() for t in (c.x, c.qweight, c.scales, c.qzeros))
    y16 = _check_gemm(sba, gpu, x, qw, s, qz, 128, 0, tag="config0")
    # row 0 alone (M = 1) equals row 0 of the M = 16 run: the kernel does not depend on M
    y1 = sba.awq_gemm(*_dev(gpu, x[:1], qw, s, qz), 0).cpu().numpy()
    assert awq_ref.rel_frobenius(y1[0], y16[0]) < 1e-3
    W = sba.awq_dequantize(*_dev(gpu, qw, s, qz)).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), awq_ref.dequantize(qw, s, qz, 128).view(np.uint16))


def test_gemm_workspace_counters_stay_zero(sba, gpu):
    from server_benchmark_amd import ops
    x, qw, s, qz = _np_case(16, 1024, 512, 128, seed=3)
    d = _dev(gpu, x, qw, s, qz)
    for _ in range(3):
        sba.awq_gemm(*d, force_split_k=4)
    torch.cuda.synchronize()
    ws = ops.get_workspace(gpu, 1)
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0


def test_split_k_exchange_is_stable_over_many_launches_and_two_streams(sba, gpu):
    """The split-K hand-off (partial tiles + arrival counters in the workspace) over a few thousand
    launches: shapes alternate on one stream and share its workspace, a second stream with a
    workspace of its own runs the same calls at the same time, and every result must carry the bits
    of the first one."""
    cases = []
    for M, K, N, seed in ((16, 4096, 2048, 1), (1, 8192, 1024, 2), (7, 2048, 264, 3), (32, 4096, 512, 4)):
        x, qw, s, qz = _np_case(M, K, N, 128, seed=seed)
        cases.append(_dev(gpu, x, qw, s, qz))
    first = [sba.awq_gemm(*c, 0).clone() for c in cases]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    outs = {0: [], 1: []}
    for it in range(400):
        for i, c in enumerate(cases):
            outs[0].append((i, sba.awq_gemm(*c, 0)))
            with torch.cuda.stream(side):
                outs[1].append((i, sba.awq_gemm(*c, 0)))
        if it % 50 == 49:               # compare in batches, so that launches queue up back to back
            torch.cuda.synchronize()
            for k in (0, 1):
                for i, y in outs[k]:
                    assert torch.equal(y, first[i]), (it, k, i)
                outs[k].clear()
    torch.cuda.synchronize()


def test_workspace_reset_zeroes_the_counters(sba, gpu):
    """A workspace whose counters were left non-zero (a call cut short) gives wrong split-K sums
    until it is reset; awqmi_workspace_reset puts it back."""
    from server_benchmark_amd import _lib
    lib = _lib.load()
    x, qw, s, qz = _np_case(16, 1024, 512, 128, seed=4)
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    nbytes = lib.awqmi_gemm_workspace_bytes(16, 1024, 512, 4)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=gpu)
    y = torch.empty((16, 512), dtype=torch.float16, device=gpu)
    st = torch.cuda.current_stream().cuda_stream

    def call():
        rc = lib.awqmi_gemm_f16(xd.data_ptr(), qwd.data_ptr(), sd.data_ptr(), qzd.data_ptr(), y.data_ptr(),
                                ws.data_ptr(), ws.numel(), 16, 1024, 512, 128, 4, st)
        assert rc == 0
        torch.cuda.synchronize()
        return y.clone()

    good = call()
    ws[:65536].view(torch.int32).fill_(-7)      # what a launch that died half-way could leave behind
    assert lib.awqmi_workspace_reset(ws.data_ptr(), ws.numel(), st) == 0
    torch.cuda.synchronize()
    assert int(ws[:65536].view(torch.int32).abs().sum().item()) == 0
    assert torch.equal(call(), good)


# ------------------------------------------------------------------ prefill GEMM (M > 16) and fallback

@pytest.mark.parametrize("M,K,N,G", [(17, 256, 256, 128), (64, 512, 512, 128), (300, 1024, 520, 128),
                                     (512, 2048, 1024, 128), (257, 192, 264, 32), (40, 256, 128, 64),
                                     (33, 384, 256, -1)])
def test_gemm_prefill(sba, gpu, M, K, N, G):
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + K)
    _check_gemm(sba, gpu, x, qw, s, qz, K if G <= 0 else G, 0, tag="prefill")


@pytest.mark.parametrize("M,K,N,G", [(65, 512, 512, 128), (100, 1024, 520, 128), (128, 2048, 1024, 128),
                                     (96, 192, 264, 32), (127, 384, 256, -1), (128, 1024, 8192 + 256, 128),
                                     (129, 512, 512, 128), (160, 1024, 520, 64), (192, 2048, 1024, 128),
                                     (190, 512, 8192 + 256, 128)])
def test_gemm_half_tile(sba, gpu, M, K, N, G):
    """65 .. 192 rows run the 128- / 192-row workgroup tile (ragged rows / columns, K split included);
    two runs agree bit for bit."""
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + K + 1)
    g = K if G <= 0 else G
    y1 = _check_gemm(sba, gpu, x, qw, s, qz, g, 0, tag="half-tile")
    y2 = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0).cpu().numpy()
    assert np.array_equal(y1.view(np.uint16), y2.view(np.uint16))


@pytest.mark.parametrize("M,K,N,G,rows", [(257, 2048, 520, 128, None), (320, 1024, 2560, 128, None),
                                          (384, 512, 10240, 64, None), (640, 1024, 1280, 128, None),
                                          (700, 256, 264, 32, None),
                                          (300, 1024, 1032, 128, 64), (300, 1024, 1032, 128, 128),
                                          (500, 1024, 1032, 128, 192), (100, 1024, 1032, 128, 256)])
def test_gemm_several_row_tiles_of_every_size(sba, gpu, M, K, N, G, rows):
    """Mid-sized batches: the library picks 64-, 128-, 192- or 256-row tiles per launch and runs
    several row tiles of the size (ragged last tile, ragged columns, K split of the last round);
    rows forces a size through the development entry point so that each one is covered."""
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + N)
    variant = None if rows is None else (rows // 64) << 20
    y1 = _check_gemm(sba, gpu, x, qw, s, qz, G, 0, tag=f"row-tiles {rows}", variant=variant)
    y2 = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0, _dev_variant=variant).cpu().numpy()
    assert np.array_equal(y1.view(np.uint16), y2.view(np.uint16))


@pytest.mark.parametrize("M,K,N", [(512, 1024, 1280), (300, 2048, 520), (2048, 512, 5120), (768, 1536, 8192 + 256)])
def test_gemm_prefill_partial_rounds(sba, gpu, M, K, N):
    """Tile counts that are not a multiple of the CU count, ragged last row / column tiles;
    two runs must agree bit for bit."""
    x, qw, s, qz = _np_case(M, K, N, 128, seed=M + N)
    y1 = _check_gemm(sba, gpu, x, qw, s, qz, 128, 0, tag="prefill-rounds")
    y2 = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0).cpu().numpy()
    assert np.array_equal(y1.view(np.uint16), y2.view(np.uint16))      # deterministic


@pytest.mark.parametrize("M,K,N,G", [(300, 1024, 520, 128), (512, 2048, 1024, 128), (257, 192, 264, 32),
                                     (700, 256, 264, 64), (1024, 512, 1280, 128), (2048, 512, 5120, 128),
                                     (768, 1536, 8192 + 256, 128), (1500, 384, 2056, -1), (4100, 320, 776, 64)])
def test_gemm_dequantise_once_form(sba, gpu, M, K, N, G):
    """The many-row form (weights dequantised once into a panel in the workspace, then the dense
    kernel fed by direct-to-LDS loads), forced through the development entry point at small
    shapes: ragged rows and columns, stage counts that are not a multiple of the ring length,
    a K split of a sparse last round, groups of 32 / 64 / 128 / K.  Checked against the oracle, and
    bit for bit against the fused kernel with 256-row tiles (same k-step order, same split)."""
    from server_benchmark_amd import _lib, ops
    lib = _lib.load()
    g = K if G <= 0 else G
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + 3 * N)
    y_dense = _check_gemm(sba, gpu, x, qw, s, qz, g, 0, tag="dense form", variant=ops.DEV_VARIANT_DENSE)
    assert lib.awqmi_dev_last_gemm_form() == _lib.FORM_DENSE
    y_fused = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0, _dev_variant=ops.DEV_VARIANT_NO_DENSE | (4 << 20)).cpu().numpy()
    assert lib.awqmi_dev_last_gemm_form() == _lib.FORM_FUSED
    assert np.array_equal(y_dense.view(np.uint16), y_fused.view(np.uint16))
    y_again = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0, _dev_variant=ops.DEV_VARIANT_DENSE).cpu().numpy()
    assert np.array_equal(y_dense.view(np.uint16), y_again.view(np.uint16))


def test_gemm_dequantise_once_default_rule_and_small_workspace(sba, gpu):
    """From 2048 rows on the public entry point takes the dequantise-once form when the workspace
    holds the panel (a row-padded qweight included) and the fused kernel when it does not; both
    return the same bits."""
    from server_benchmark_amd import _lib, ops
    lib = _lib.load()
    M, K, N, G = 2048, 256, 1024 * 8, 128
    x, qw, s, qz = _np_case(M, K, N, G, seed=11)
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    y = sba.awq_gemm(xd, qwd, sd, qzd, 0)
    assert lib.awqmi_dev_last_gemm_form() == _lib.FORM_DENSE
    padded = ops.pad_qweight_rows(qwd)
    assert not padded.is_contiguous()
    y_pad = sba.awq_gemm(xd, padded, sd, qzd, 0)
    assert lib.awqmi_dev_last_gemm_form() == _lib.FORM_DENSE
    assert torch.equal(y, y_pad)
    # a workspace without room for the panel: the same call runs the fused kernel
    small = torch.zeros(lib.awqmi_gemm_workspace_bytes(1024, K, N, 0), dtype=torch.uint8, device=gpu)
    y_small = torch.empty_like(y)
    st = lib.awqmi_gemm_f16(xd.data_ptr(), qwd.data_ptr(), sd.data_ptr(), qzd.data_ptr(), y_small.data_ptr(),
                            small.data_ptr(), small.numel(), M, K, N, G, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 0 and lib.awqmi_dev_last_gemm_form() == _lib.FORM_FUSED
    torch.cuda.synchronize()
    assert torch.equal(y, y_small)
    ref = awq_ref.gemm_wide(x[:64], qw, s, qz, G)
    assert awq_ref.rel_frobenius(y[:64].cpu().numpy(), ref) <= TOL
    # the same row count on a narrow layer (64 tiles of 256 x 256): the fused kernel's smaller row tiles
    # fill the chip better, so the default stays with it; from 4096 rows on the form is taken again
    for rows, form in ((2048, _lib.FORM_FUSED), (4096, _lib.FORM_DENSE)):
        xn, qwn, sn, qzn = _np_case(rows, K, 2048, G, seed=12)
        xnd, qwnd, snd, qznd = _dev(gpu, xn, qwn, sn, qzn)
        yn = sba.awq_gemm(xnd, qwnd, snd, qznd, 0)
        assert lib.awqmi_dev_last_gemm_form() == form
        refn = awq_ref.gemm_wide(xn[-64:], qwn, sn, qzn, G)
        assert awq_ref.rel_frobenius(yn[-64:].cpu().numpy(), refn) <= TOL


def test_gemm_dequantise_once_form_replays_from_a_graph(sba, gpu):
    """The many-row form is three plain launches (panel pass, dense kernel, K-split sum) on the
    caller's stream and workspace: captured once, every replay -- with new activations and with
    eager calls of other shapes on the same stream in between -- equals the eager result."""
    from server_benchmark_amd import _lib
    lib = _lib.load()
    M, K, N, G = 2304, 320, 1032 * 8, 64          # 9 x 33 tiles: a sparse last round, split in K; ragged N
    x, qw, s, qz = _np_case(M, K, N, G, seed=21)
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        eager = sba.awq_gemm(xd, qwd, sd, qzd, 0)            # sizes this stream's workspace
        assert lib.awqmi_dev_last_gemm_form() == _lib.FORM_DENSE
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            y = sba.awq_gemm(xd, qwd, sd, qzd, 0)
        for rep in range(3):
            if rep:
                xd.copy_(torch.randn((M, K), device=gpu, generator=torch.Generator(device=gpu).manual_seed(rep)).half())
                eager = sba.awq_gemm(xd, qwd, sd, qzd, 0)
            sba.awq_gemm(xd[:5], qwd, sd, qzd, 0)           # a skinny call on the same workspace in between
            y.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager)
    torch.cuda.current_stream().wait_stream(st)
    ref = awq_ref.gemm_wide(xd[:32].cpu().numpy(), qw, s, qz, G)
    assert awq_ref.rel_frobenius(y[:32].cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("M,K,N,G", [(3, 96, 40, 32), (20, 100, 16, 50), (2, 24, 8, 8)])
def test_gemm_generic_fallback(sba, gpu, M, K, N, G):
    x, qw, s, qz = _np_case(M, K, N, G, seed=5)
    _check_gemm(sba, gpu, x, qw, s, qz, G, 0, tag="generic")


def test_more_rows_than_one_grid_dimension_holds(sba, gpu):
    """Shapes whose row count exceeds 65535, the limit of a grid's second dimension: the
    dequantize launch (one row per slab when the group size is odd) and the any-shape GEMM
    run as consecutive slabs."""
    _, qw, s, qz = _np_case(1, 70001, 8, 1, seed=11)
    want = awq_ref.dequantize(qw, s, qz, 1)
    got = sba.awq_dequantize(*_dev(gpu, qw, s, qz), 0, 0, 0).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    x, qw, s, qz = _np_case(70001, 24, 8, 8, seed=12)
    _check_gemm(sba, gpu, x, qw, s, qz, 8, 0, tag="generic-tall")


def test_bad_arguments_raise_without_launch(sba, gpu):
    x, qw, s, qz = _dev(gpu, *_np_case(2, 256, 64, 128, seed=1))
    with pytest.raises(ValueError):
        sba.awq_gemm(x[:, :128].contiguous(), qw, s, qz, 0)
    with pytest.raises(ValueError):
        sba.awq_gemm(x.float(), qw, s, qz, 0)
    with pytest.raises(ValueError):
        sba.awq_gemm(x.cpu(), qw, s, qz, 0)
    with pytest.raises(ValueError):
        sba.awq_dequantize(qw, s[:, :32].contiguous(), qz)


def test_linear_method_apply(sba, gpu):
    cfg = sba.AWQConfig.from_config({"w_bit": 4, "q_group_size": 128, "zero_point": True})
    layer = torch.nn.Module()
    m = cfg.get_quant_method(layer, "model.layers.0.mlp.down_proj")
    m.create_weights(layer, 512, [128, 128], 512, 256, torch.float16, device=gpu)
    x, qw, s, qz = _np_case(6, 512, 256, 128, seed=9)
    sd = {"qweight": torch.from_numpy(qw), "qzeros": torch.from_numpy(qz), "scales": torch.from_numpy(s)}
    layer.load_state_dict(sd)
    m.process_weights_after_loading(layer)
    xin = torch.from_numpy(x).to(gpu).reshape(2, 3, 512)
    bias = torch.linspace(-1, 1, 256, dtype=torch.float16, device=gpu)
    y = m.apply(layer, xin, bias)
    assert y.shape == (2, 3, 256)
    ref = awq_ref.gemm_wide(x, qw, s, qz, 128) + bias.cpu().numpy().astype(np.float64)
    assert awq_ref.rel_frobenius(y.reshape(6, 256).cpu().numpy(), ref) <= TOL


def test_gemm_random_shapes_across_dispatch_boundaries(sba, gpu):
    """Seeded random (M, K, N, G) around every boundary of the kernel choice (16 / 32 / 48 / 64 /
    128 / 192 / 256 rows, odd word counts, ragged tiles, K-split on and off), against the oracle."""
    rng = np.random.default_rng(2024)
    ms = [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 127, 128, 129, 191, 192, 193, 255, 256, 257, 300]
    worst = 0.0
    for case in range(40):
        M = int(ms[case % len(ms)]) if case < len(ms) else int(rng.integers(1, 320))
        G = int(rng.choice([32, 64, 128, 256]))
        K = int(rng.integers(1, 9)) * 256
        N = int(rng.integers(1, 150)) * 8
        x, qw, s, qz = _np_case(M, K, N, G, seed=1000 + case)
        y = sba.awq_gemm(*_dev(gpu, x, qw, s, qz), 0).cpu().numpy()
        ref = awq_ref.gemm_wide(x, qw, s, qz, G)
        err = awq_ref.rel_frobenius(y, ref)
        assert err <= TOL, f"M={M} K={K} N={N} G={G}: rel_fro={err:.3e}"
        worst = max(worst, err)
    print(f"[random shapes] worst rel_fro={worst:.2e}", flush=True)


def _with_pitch(qw_dev, extra_words):
    """The same qweight as a view of a buffer whose rows are extra_words further apart; the pad
    holds a pattern that would show up in the result if it were ever read."""
    K, NW = qw_dev.shape
    width = (NW + extra_words + 3) // 4 * 4          # a row pitch must keep 16-byte groups whole
    buf = torch.full((K, width), 0x5A5A5A5A, dtype=torch.int32, device=qw_dev.device)
    v = buf[:, :NW]
    v.copy_(qw_dev)
    return v


@pytest.mark.parametrize("M,K,N,G,pitch,split", [
    (1, 1024, 2048, 128, 32, 0), (16, 1024, 2048, 128, 32, 0), (5, 4096, 2048, 128, 32, 3),     # skinny, tail form
    (16, 2048, 264, 64, 4, 0), (3, 512, 136, 256, 12, 2), (7, 256, 8, 32, 36, 0),                 # other groups, one word per lane
    (24, 12288, 512, 128, 32, 0), (32, 3072, 2048, 64, 32, 1), (48, 1024, 2048, 128, 32, 0),    # 32-row passes, LDS ring
    (64, 512, 2048, 128, 32, 0), (100, 1024, 520, 128, 8, 0), (300, 2048, 2048, 128, 32, 0),    # MFMA tiles
    (700, 1024, 2064, 32, 4, 0), (512, 1024, 4096, 128, 32, 0),
    (3, 96, 40, 32, 4, 0), (20, 100, 16, 50, 8, 0)])                                              # generic kernel
def test_qweight_with_a_row_pitch(sba, gpu, M, K, N, G, pitch, split):
    """qweight rows `pitch` words further apart than a row is long (what
    AWQLinearMethod.process_weights_after_loading hands over for rows that are a multiple of 1 KiB):
    awq_gemm on every kernel and awq_dequantize give the bits of the contiguous tensor, and match
    the oracle; the pad is never read."""
    x, qw, s, qz = _np_case(M, K, N, G, seed=M + K + N)
    g = K if G <= 0 else G
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    qwp = _with_pitch(qwd, pitch)
    assert not qwp.is_contiguous() and qwp.stride(0) >= N // 8 + pitch
    y0 = sba.awq_gemm(xd, qwd, sd, qzd, force_split_k=split)
    y1 = sba.awq_gemm(xd, qwp, sd, qzd, force_split_k=split)
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    ref = awq_ref.gemm_wide(x, qw, s, qz, g)
    assert awq_ref.rel_frobenius(y1.cpu().numpy(), ref) <= TOL
    W0 = sba.awq_dequantize(qwd, sd, qzd)
    W1 = sba.awq_dequantize(qwp, sd, qzd)
    assert torch.equal(W0.view(torch.int16), W1.view(torch.int16))
    Wref = awq_ref.dequantize(qw, s, qz, g)
    assert np.array_equal(W1.cpu().numpy().view(np.uint16), Wref.view(np.uint16))


def test_qweight_pitch_is_validated(sba, gpu):
    x, qw, s, qz = _np_case(4, 256, 256, 128, seed=1)
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    bad = torch.zeros((256, 34), dtype=torch.int32, device=gpu)[:, :32]      # pitch not a multiple of 4 words
    with pytest.raises(ValueError):
        sba.awq_gemm(xd, bad, sd, qzd)
    with pytest.raises(ValueError):
        sba.awq_gemm(xd, qwd.t().contiguous().t(), sd, qzd)      # column-major


def test_linear_method_pads_kib_rows_and_matches_contiguous(sba, gpu):
    """A layer whose packed rows are 32 lines: process_weights_after_loading re-pitches qweight,
    apply gives the bits of awq_gemm on the contiguous tensor at decode and prefill sizes."""
    cfg = sba.AWQConfig(4, 128, True)
    m = sba.AWQLinearMethod(cfg)
    layer = torch.nn.Module()
    m.create_weights(layer, 512, [8192], 512, 8192, torch.float16, device=gpu)
    x, qw, s, qz = _np_case(300, 512, 8192, 128, seed=77)
    layer.load_state_dict({"qweight": torch.from_numpy(qw), "qzeros": torch.from_numpy(qz),
                           "scales": torch.from_numpy(s)})
    m.process_weights_after_loading(layer)
    assert layer.qweight.stride() == (1056, 1)
    xd, qwd, sd, qzd = _dev(gpu, x, qw, s, qz)
    for rows in (1, 16, 40, 300):
        y = m.apply(layer, xd[:rows].contiguous())
        y0 = sba.awq_gemm(xd[:rows].contiguous(), qwd, sd, qzd)
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16))
