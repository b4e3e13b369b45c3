"""The allocation-free entry point awqmi_gemm_f16_noalloc (split-K counters and partial tiles in
a static device array inside the library) against awqmi_gemm_f16 with a caller-owned workspace,
through the C ABI: bit-identical outputs on calls in a row that share the array, the later ones
smaller than the first; no device allocation during the calls; sizes beyond the array refused
before any launch.  Collected last on purpose: it is the newest entry point, and a failure here
must not hide the rest of the suite."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SCRATCH_LIMIT = 8
STATIC_BYTES = 65536 + (16 << 20)


def _case(M, K, N, G, gpu, seed):
    g = torch.Generator(device=gpu).manual_seed(seed)
    qw = torch.randint(-2 ** 31, 2 ** 31, (K, N // 8), dtype=torch.int32, device=gpu, generator=g)
    qz = torch.randint(-2 ** 31, 2 ** 31, (K // G, N // 8), dtype=torch.int32, device=gpu, generator=g)
    sc = (torch.rand((K // G, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    x = torch.randn((M, K), device=gpu, generator=g).half()
    return x, qw, sc, qz


def _both(lib, gpu, M, K, N, G, split, seed):
    """(noalloc output, workspace output, device bytes allocated by the noalloc call)"""
    x, qw, sc, qz = _case(M, K, N, G, gpu, seed)
    y_ws = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    y_na = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    # the comparison call gets a zeroed workspace of the static array's size (for the decode-sized
    # cases that is at least what the library asks for, i.e. the full-workspace result)
    need = lib.awqmi_gemm_workspace_bytes(M, K, N, split)
    assert need <= STATIC_BYTES or M > 32
    ws = torch.zeros(STATIC_BYTES, dtype=torch.uint8, device=gpu)
    st = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    print(f"[noalloc] M={M} K={K} N={N} G={G} split={split} needs {need} scratch bytes", flush=True)
    before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    rc = lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qw.data_ptr(), 0, sc.data_ptr(), qz.data_ptr(), y_na.data_ptr(),
                                    M, K, N, G, split, st)
    assert rc == 0, lib.awqmi_status_string(rc).decode()
    torch.cuda.synchronize()
    after = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    rc = lib.awqmi_gemm_f16(x.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), y_ws.data_ptr(),
                            ws.data_ptr(), ws.numel(), M, K, N, G, split, st)
    assert rc == 0, lib.awqmi_status_string(rc).decode()
    torch.cuda.synchronize()
    assert before == after
    # and against the dequantize kernel + a library matmul, so that "equal" cannot mean "equally wrong"
    W = torch.empty((K, N), dtype=torch.float16, device=gpu)
    assert lib.awqmi_dequantize_f16(qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), W.data_ptr(), K, N, G, st) == 0
    ref = x.float() @ W.float()
    err = float((y_na.float() - ref).norm() / ref.norm())
    assert err <= 2e-3, err
    return y_na, y_ws


def test_noalloc_gemm_matches_workspace_gemm_on_calls_in_a_row(gpu):
    from server_benchmark_amd import _lib
    lib = _lib.load()
    # decode-sized calls whose split-K sums go through the static array (8 parts, then 6 of a
    # ragged width, then a forced split on a small layer), each smaller than the one before;
    # then the MFMA kernel with a K split that fits the array (partial tiles of 256 KiB) and one
    # that does not (every tile on one workgroup), and a call with no split at all
    calls = [(16, 8192, 8192, 128, 0, 1), (4, 8192, 2048 + 264, 128, 0, 2), (3, 1024, 512, 128, 4, 3),
             (1, 1024, 512, 128, 4, 4), (100, 2048, 520, 128, 0, 5), (300, 2048, 1024, 128, 0, 5),
             (16, 512, 59136, 128, 0, 6), (5, 256, 264, 64, 2, 7)]
    for M, K, N, G, split, seed in calls:
        y_na, y_ws = _both(lib, gpu, M, K, N, G, split, seed)
        assert torch.isfinite(y_na).all()
        assert torch.equal(y_na.view(torch.int16), y_ws.view(torch.int16)), (M, K, N, split)
    # the same first call again after the smaller ones: stale partial tiles of the calls between
    # must not leak into it
    y_na, y_ws = _both(lib, gpu, *calls[0])
    assert torch.equal(y_na.view(torch.int16), y_ws.view(torch.int16))


def test_noalloc_gemm_refuses_what_does_not_fit(gpu):
    from server_benchmark_amd import _lib
    lib = _lib.load()
    M, K, N, G = 16, 8192, 8192, 128
    x, qw, sc, qz = _case(M, K, N, G, gpu, 9)
    y = torch.zeros((M, N), dtype=torch.float16, device=gpu)
    st = torch.cuda.current_stream().cuda_stream
    # a forced split of 64 on this width wants 64 x 32 x 8192 fp32 partials = 64 MiB
    assert lib.awqmi_gemm_workspace_bytes(M, K, N, 64) > STATIC_BYTES
    rc = lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qw.data_ptr(), 0, sc.data_ptr(), qz.data_ptr(), y.data_ptr(),
                                    M, K, N, G, 64, st)
    assert rc == SCRATCH_LIMIT
    assert "static" in lib.awqmi_status_string(rc).decode()
    torch.cuda.synchronize()
    assert not y.any()                      # nothing was launched
    # ordinary validation still comes first
    assert lib.awqmi_gemm_f16_noalloc(0, qw.data_ptr(), 0, sc.data_ptr(), qz.data_ptr(), y.data_ptr(),
                                      M, K, N, G, 0, st) == 6
    assert lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qw.data_ptr(), 0, sc.data_ptr(), qz.data_ptr(), y.data_ptr(),
                                      M, K, N + 4, G, 0, st) == 1


def test_noalloc_gemm_replays_from_a_captured_graph(gpu):
    """What the entry point is for: a call recorded into a HIP graph with no workspace to carry.
    Replays, with other calls of the entry point and eager work in between, must reproduce the
    eager result bit for bit."""
    from server_benchmark_amd import _lib
    lib = _lib.load()
    assert lib.awqmi_init() == 0                      # set-up outside the capture
    M, K, N, G = 8, 4096, 2048, 128
    x, qw, sc, qz = _case(M, K, N, G, gpu, 11)
    y_eager = torch.empty((M, N), dtype=torch.float16, device=gpu)
    y_graph = torch.zeros((M, N), dtype=torch.float16, device=gpu)

    def call(y, stream):
        rc = lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qw.data_ptr(), 0, sc.data_ptr(), qz.data_ptr(), y.data_ptr(),
                                        M, K, N, G, 0, stream)
        assert rc == 0, lib.awqmi_status_string(rc).decode()

    assert lib.awqmi_gemm_auto_split_k(M, K, N, G) > 1            # the scratch array is really in use
    call(y_eager, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            call(y_graph, s.cuda_stream)
        for _ in range(3):
            y_graph.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_graph.view(torch.int16), y_eager.view(torch.int16))
            other, _ = _both(lib, gpu, 3, 1024, 512, 128, 4, 12)       # eager calls on the same array in between
            assert torch.isfinite(other).all()
    torch.cuda.current_stream().wait_stream(s)


def test_noalloc_gemm_takes_the_methods_row_padded_qweight(gpu):
    """The layout AWQLinearMethod keeps after loading (rows one 128-byte line further apart) through
    the allocation-free entry point and through its Python wrapper: the bits of the contiguous
    tensor through awqmi_gemm_f16, on two calls in a row (the second with fewer rows)."""
    from server_benchmark_amd import _lib, ops
    lib = _lib.load()
    assert lib.awqmi_init() == 0
    K, N, G = 1024, 8192, 128
    for M in (16, 3):
        x, qw, sc, qz = _case(M, K, N, G, gpu, 40 + M)
        qwp = ops.pad_qweight_rows(qw)
        assert not qwp.is_contiguous() and qwp.stride(0) == N // 8 + 32
        ws = torch.zeros(STATIC_BYTES, dtype=torch.uint8, device=gpu)
        st = torch.cuda.current_stream().cuda_stream
        y_ws = torch.empty((M, N), dtype=torch.float16, device=gpu)
        assert lib.awqmi_gemm_f16(x.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), y_ws.data_ptr(),
                                  ws.data_ptr(), ws.numel(), M, K, N, G, 0, st) == 0
        y_c = torch.empty_like(y_ws)
        assert lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qwp.data_ptr(), qwp.stride(0), sc.data_ptr(), qz.data_ptr(),
                                          y_c.data_ptr(), M, K, N, G, 0, st) == 0
        y_py = ops.awq_gemm_noalloc(x, qwp, sc, qz, torch.empty_like(y_ws))
        torch.cuda.synchronize()
        assert torch.equal(y_ws, y_c) and torch.equal(y_ws, y_py)
    # a pitch that is no multiple of 16 bytes is refused before anything is launched
    assert lib.awqmi_gemm_f16_noalloc(x.data_ptr(), qw.data_ptr(), N // 8 + 1, sc.data_ptr(), qz.data_ptr(),
                                      y_c.data_ptr(), M, K, N, G, 0, st) != 0
