"""CPU-only checks of the host side: the C-ABI library loads and exports every symbol the
header declares, host-side validation rejects bad calls before any launch, the layer
methods register the right parameters, and the workload generators produce the stated
shapes and byte counts.  No compute call is made (no GPU here)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from server_benchmark_amd import _lib
    return _lib.load()


def test_library_exports_every_declared_symbol(lib):
    from server_benchmark_amd import _lib
    hdr = ""
    for name in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if name.endswith(".h"):
            hdr += open(os.path.join(ROOT, "include", name)).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(awqmi_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 14
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert lib.awqmi_version() == 300


def test_status_strings(lib):
    seen = {lib.awqmi_status_string(i).decode() for i in range(9)}
    assert len(seen) == 9 and "ok" in seen
    assert lib.awqmi_status_string(99).decode() == "unknown status"


def test_validation_happens_before_any_launch(lib):
    fake = 0x1000   # non-null, 16-byte aligned, never dereferenced on these paths
    odd = 0x1008
    # null pointers
    assert lib.awqmi_dequantize_f16(0, fake, fake, fake, 128, 64, 128, 0) == 6
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, 0, 0, 0, 1, 128, 64, 128, 0, 0) == 6
    # shape relations: N % 8, K % group, positive sizes
    assert lib.awqmi_dequantize_f16(fake, fake, fake, fake, 128, 60, 128, 0) == 1
    assert lib.awqmi_dequantize_f16(fake, fake, fake, fake, 100, 64, 48, 0) == 1
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, fake, 0, 0, 0, 128, 64, 128, 0, 0) == 1
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, fake, 0, 0, 4, 128, 64, 96, 0, 0) == 1
    # alignment
    assert lib.awqmi_dequantize_f16(fake, odd, fake, fake, 128, 64, 128, 0) == 2
    assert lib.awqmi_gemm_f16(odd, fake, fake, fake, fake, 0, 0, 4, 128, 64, 128, 0, 0) == 2
    # split_k range, missing / short workspace
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, fake, 0, 0, 4, 1024, 64, 128, 65, 0) == 7
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, fake, 0, 0, 4, 1024, 64, 128, 2, 0) == 6
    assert lib.awqmi_gemm_f16(fake, fake, fake, fake, fake, fake, 1000, 4, 1024, 64, 128, 2, 0) == 3
    # MoE entry points
    assert lib.awqmi_moe_align(0, 8, 4, 16, fake, fake, fake, 0) == 6
    assert lib.awqmi_moe_align(fake, 8, 2000, 16, fake, fake, fake, 0) == 7
    assert lib.awqmi_moe_topk_softmax_f32(fake, 4, 8, 9, 1, fake, fake, 0) == 7
    assert lib.awqmi_moe_gemm_f16(fake, fake, fake, fake, fake, fake, fake, fake, 0, 8, 2, 16, 4, 100, 64, 50,
                                  0, 0, 0, 0) == 4
    assert lib.awqmi_moe_gemm_f16(fake, fake, fake, fake, fake, fake, fake, fake, 0, 8, 2, 24, 4, 128, 64, 128,
                                  0, 0, 0, 0) == 7
    # block rows of the MFMA form: 64 / 128 / 256 are accepted (so a bad group size is what is
    # reported), 48 or 512 are not; the query sizes only the counters for them
    for tile, want in ((64, 4), (128, 4), (256, 4), (48, 7), (512, 7)):
        assert lib.awqmi_moe_gemm_f16(fake, fake, fake, fake, fake, fake, fake, fake, 0, 8, 2, tile, 4, 100, 64,
                                      50, 0, 0, 0, 0) == want
    assert lib.awqmi_moe_gemm_workspace_bytes(4096, 8, 1024, 1024, 0, 128) == 65536
    assert lib.awqmi_moe_gemm_workspace_bytes(4096, 8, 1024, 1024, 0, 48) == 0
    assert lib.awqmi_silu_and_mul_f16(fake, fake, 4, 12, 0) == 1
    assert lib.awqmi_moe_sum_f16(fake, fake, 4, 2, 12, 0) == 1
    # whole-block MoE call: null operand, top-k beyond E, short workspace
    ok = [fake] * 9
    assert lib.awqmi_fused_moe_f16(*ok[:8], 0, 4, 256, 128, 8, 2, 128, 1, fake, 1 << 30, 0) == 6
    assert lib.awqmi_fused_moe_f16(*ok, 4, 256, 128, 8, 9, 128, 1, fake, 1 << 30, 0) == 7
    assert lib.awqmi_fused_moe_f16(*ok, 4, 256, 128, 8, 2, 128, 1, fake, 1024, 0) == 3
    # routed form: a bias with softmax scoring, an unknown scoring id
    okr = [fake, fake, fake] + [fake] * 7
    assert lib.awqmi_fused_moe_routed_f16(*okr, 4, 256, 128, 8, 2, 128, 0, 1, 1.0, fake, 1 << 30, 0) == 7
    okr[2] = 0
    assert lib.awqmi_fused_moe_routed_f16(*okr, 4, 256, 128, 8, 2, 128, 2, 1, 1.0, fake, 1 << 30, 0) == 7
    assert lib.awqmi_fused_moe_routed_f16(*okr, 4, 256, 128, 8, 2, 128, 1, 1, 2.5, fake, 1024, 0) == 3
    assert lib.awqmi_fused_moe_f16(*ok, 4, 250, 128, 8, 2, 128, 1, fake, 1 << 30, 0) == 1


def test_workspace_reset_and_dev_entry_points_validate_on_the_host(lib):
    fake, odd = 0x1000, 0x1008
    assert lib.awqmi_workspace_reset(0, 1 << 20, 0) == 6
    assert lib.awqmi_workspace_reset(odd, 1 << 20, 0) == 2
    assert lib.awqmi_workspace_reset(fake, 65535, 0) == 3
    # the development entry points are the public ones plus a variant argument: same checks,
    # and the variant of one call is gone when the call returns (the query that follows sees
    # the default rules again)
    assert lib.awqmi_dev_gemm_f16(fake, fake, fake, fake, 0, 0, 0, 1, 128, 64, 128, 0, 0, 1) == 6
    assert lib.awqmi_dev_gemm_f16(fake, fake, fake, fake, fake, 0, 0, 4, 1024, 64, 128, 65, 0, 1 << 23) == 7
    big = (4096, 2048, 768, 128, 8, 128)
    rows = lib.awqmi_fused_moe_block_rows(*big)
    assert lib.awqmi_dev_fused_moe_block_rows(*big, 2048) == 16
    assert lib.awqmi_dev_fused_moe_block_rows(*big, 2 << 16) == 128
    assert lib.awqmi_dev_fused_moe_block_rows(*big, -1) == rows
    assert lib.awqmi_fused_moe_block_rows(*big) == rows


def test_row_pitch_entry_points_validate_on_the_host(lib):
    """awqmi_gemm_ld_f16 / awqmi_dequantize_ld_f16: the row pitch must cover a row and keep 16-byte
    groups whole; everything else is checked as in the contiguous calls, before any launch."""
    fake = 0x1000
    assert lib.awqmi_gemm_ld_f16(fake, fake, 15, fake, fake, fake, 0, 0, 4, 1024, 128, 128, 0, 0) == 7   # pitch < N / 8
    assert lib.awqmi_gemm_ld_f16(fake, fake, 18, fake, fake, fake, 0, 0, 4, 1024, 128, 128, 0, 0) == 7   # not % 4
    assert lib.awqmi_gemm_ld_f16(fake, 0, 48, fake, fake, fake, 0, 0, 4, 1024, 128, 128, 0, 0) == 6
    assert lib.awqmi_gemm_ld_f16(fake, fake, 48, fake, fake, fake, 0, 0, 4, 1000, 128, 128, 0, 0) == 1
    assert lib.awqmi_dequantize_ld_f16(fake, 12, fake, fake, fake, 128, 128, 128, 0) == 7
    assert lib.awqmi_dequantize_ld_f16(fake, 48, fake, fake, 0, 128, 128, 128, 0) == 6


def test_pad_qweight_rows_and_the_method_hook(sba):
    """A packed row of 32 lines or more that is a multiple of 512 bytes gets one 128-byte line of
    pitch more (same shape, same values, a view of a wider buffer); any other row length is left
    alone.  AWQLinearMethod.process_weights_after_loading applies it and keeps qzeros / scales
    contiguous."""
    import importlib
    ops = importlib.import_module(sba.__name__ + ".ops")
    g = torch.Generator().manual_seed(0)
    q = torch.randint(-2**31, 2**31 - 1, (16, 1024), dtype=torch.int32, generator=g)      # 32 lines
    p = ops.pad_qweight_rows(q)
    assert tuple(p.shape) == (16, 1024) and p.stride() == (1056, 1) and torch.equal(p, q)
    assert not p.is_contiguous() and p.data_ptr() != q.data_ptr()
    q4 = torch.randint(-2**31, 2**31 - 1, (8, 1152), dtype=torch.int32, generator=g)      # 36 lines: multiple of 4
    assert ops.pad_qweight_rows(q4).stride() == (1184, 1)
    for shape in ((16, 1056), (16, 1120), (64, 256), (64, 640)):                           # 33 / 35 / 8 / 20 lines
        t = torch.zeros(shape, dtype=torch.int32)
        assert ops.pad_qweight_rows(t) is t
    assert ops.pad_qweight_rows(p) is p                                                     # already padded
    m = sba.AWQLinearMethod(sba.AWQConfig(4, 128, True))
    layer = torch.nn.Module()
    m.create_weights(layer, 128, [8192], 128, 8192, torch.float16)
    layer.qweight.data.copy_(torch.randint(-2**31, 2**31 - 1, (128, 1024), dtype=torch.int32, generator=g))
    want = layer.qweight.data.clone()
    m.process_weights_after_loading(layer)
    assert layer.qweight.stride() == (1056, 1) and torch.equal(layer.qweight.data, want)
    assert layer.qzeros.is_contiguous() and layer.scales.is_contiguous()
    assert sorted(n for n, _ in layer.named_parameters()) == ["qweight", "qzeros", "scales"]


def test_fused_moe_workspace_covers_every_intermediate(lib):
    T, H, I, E, topk = 16, 2048, 768, 128, 8
    n = T * topk
    total = lib.awqmi_fused_moe_workspace_bytes(T, H, I, E, topk)
    payloads = []
    for tile in (16, 64, 128, 256):      # the call picks the block rows itself; any choice must fit
        g = max(lib.awqmi_moe_gemm_workspace_bytes(n, E, H, 2 * I, 0, tile),
                lib.awqmi_moe_gemm_workspace_bytes(n, E, I, H, 0, tile))
        cap = lib.awqmi_moe_align_capacity(n, E, tile)
        payloads.append(g + 2 * n * 4 + cap * 4 + cap // tile * 4 + 4 + n * 2 * I * 2 + n * I * 2 + n * H * 2
                        + 64 * E * 4)        # + the per-part table of the multi-workgroup align
    assert max(payloads) <= total <= max(payloads) + 10 * 256
    assert lib.awqmi_fused_moe_workspace_bytes(0, H, I, E, topk) == 0
    assert lib.awqmi_fused_moe_workspace_bytes(T, H, 100, E, topk) == 0


def test_init_without_a_gpu_reports_a_launch_failure(lib):
    """awqmi_init needs a device; without one it returns a status (no abort, no exception)."""
    import torch
    st = lib.awqmi_init()
    if torch.cuda.is_available():
        assert st == 0
    else:
        assert st == 5 and lib.awqmi_last_hip_error() != 0
        assert b"launch" in lib.awqmi_status_string(st).lower()


def test_fused_moe_block_rows(lib):
    """Block rows the one-call MoE entry picks: the skinny kernel's 16 for decode-sized batches,
    the MFMA kernel's 64 / 128 / 256 where measurements favoured them (points of the fit)."""
    q = lib.awqmi_fused_moe_block_rows
    for T in (1, 16, 128, 512, 1024, 2048):
        assert q(T, 2048, 768, 128, 8, 128) == 16
    assert q(3072, 2048, 768, 128, 8, 128) == 256
    assert q(8192, 2048, 768, 128, 8, 128) == 256
    assert q(512, 6144, 2560, 160, 8, 128) == 16
    assert q(1024, 6144, 2560, 160, 8, 128) == 64
    assert q(1024, 2048, 1408, 64, 6, 128) == 128
    assert q(2048, 6144, 2560, 160, 8, 128) == 128
    assert q(8192, 6144, 2560, 160, 8, 128) == 256
    assert q(64, 4096, 14336, 8, 2, 128) == 16
    assert q(1024, 4096, 14336, 8, 2, 128) in (128, 256)
    assert q(4096, 2048, 776, 128, 8, 128) == 16       # inter no multiple of 128: MFMA form not available
    assert q(0, 2048, 768, 128, 8, 128) == 0 and q(4, 2048, 768, 128, 200, 128) == 0
    for T in (1, 100, 5000):                           # every choice fits the workspace the query sizes
        assert lib.awqmi_fused_moe_workspace_bytes(T, 2048, 768, 128, 8) > 0


def test_workspace_and_split_k_queries(lib):
    for M, K, N in [(1, 8192, 10240), (16, 8192, 8192), (16, 8192, 59136), (4, 29568, 8192), (8, 4096, 4096)]:
        s = lib.awqmi_gemm_auto_split_k(M, K, N, 128)
        assert 1 <= s <= 64 and s <= K // 128
        need = lib.awqmi_gemm_workspace_bytes(M, K, N, 0)
        assert need == lib.awqmi_gemm_workspace_bytes(M, K, N, s)
        assert need >= 65536
        if s > 1:
            assert need >= 65536 + s * 16 * N * 4
    assert lib.awqmi_gemm_workspace_bytes(1024, 8192, 16384, 0) == 65536    # whole rounds: no partials
    # from 2048 rows on: room for the fp16 panel of the dequantise-once form (K * N * 2 bytes for
    # whole 256-column tiles) behind the counters
    assert lib.awqmi_gemm_workspace_bytes(8192, 8192, 8192, 0) == 65536 + 8192 * 8192 * 2
    assert lib.awqmi_gemm_workspace_bytes(4096, 8192, 8192 + 8, 0) >= 65536 + 8192 * (8192 + 256) * 2
    assert lib.awqmi_dev_gemm_dense_workspace_bytes(8192, 8192, 8192) == 65536 + 8192 * 8192 * 2
    # 2048 .. 4095 rows on a narrow layer (fewer than 192 tiles of 256 x 256): the fused kernel, no panel
    assert lib.awqmi_gemm_workspace_bytes(2048, 4096, 2048, 0) == 65536 + 64 * 4 * 256 * 256 * 4   # K-split partials only
    assert lib.awqmi_gemm_workspace_bytes(4096, 4096, 2048, 0) == lib.awqmi_dev_gemm_dense_workspace_bytes(4096, 4096, 2048)
    assert lib.awqmi_dev_gemm_dense_workspace_bytes(300, 1000, 512) == 0    # K no multiple of 64
    assert lib.awqmi_gemm_workspace_bytes(512, 8192, 8192, 0) == 65536 + 64 * 4 * 256 * 256 * 4   # K split
    assert lib.awqmi_gemm_auto_split_k(512, 8192, 8192, 128) == 1
    assert lib.awqmi_gemm_workspace_bytes(32, 8192, 8192, 8) >= 65536 + 8 * 32 * 8192 * 4
    assert lib.awqmi_moe_align_capacity(8, 128, 16) == (8 + 128 * 15 + 15) // 16 * 16
    assert lib.awqmi_moe_align_capacity(4096, 128, 16) % 16 == 0


def test_ops_reject_cpu_tensors_and_bad_dtypes(sba):
    c = sba.workloads.make_linear_case(2, 256, 64, 128, seed=0)
    with pytest.raises(ValueError, match="GPU"):
        sba.awq_gemm(c.x, c.qweight, c.scales, c.qzeros, 0)
    with pytest.raises(ValueError, match="GPU"):
        sba.awq_dequantize(c.qweight, c.scales, c.qzeros, 0, 0, 0)
    with pytest.raises(ValueError):
        sba.awq_gemm(c.x.float(), c.qweight, c.scales, c.qzeros, 0)
    with pytest.raises(TypeError):
        sba.awq_gemm(c.x.numpy(), c.qweight, c.scales, c.qzeros, 0)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from server_benchmark_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU or eager fallback"):
        _lib.load()


# ------------------------------------------------------------------ AWQConfig / layer methods

@pytest.mark.parametrize("cfg,want", [
    ({"w_bit": 4, "q_group_size": 128, "zero_point": True}, (4, 128, True)),
    ({"bits": 4, "group_size": 64, "zero_point": False}, (4, 64, False)),
    ({"bits": 4, "group_size": -1, "zero_point": True, "modules_to_not_convert": ["lm_head"]}, (4, -1, True)),
])
def test_awq_config_aliases(sba, cfg, want):
    c = sba.AWQConfig.from_config(cfg)
    assert (c.weight_bits, c.group_size, c.zero_point) == want
    assert c.pack_factor == 8 and c.get_name() == "awq"
    assert torch.float16 in c.get_supported_act_dtypes()


def test_awq_config_static_surface(sba):
    cfg = sba.AWQConfig
    assert cfg.get_name() == "awq" and cfg.get_min_capability() == 75
    assert cfg.get_config_filenames() == ["quant_config.json", "quantize_config.json"]
    assert "gelu" in cfg.get_scaled_act_names()


def test_awq_config_rejects(sba):
    with pytest.raises(ValueError):
        sba.AWQConfig.from_config({"bits": 8, "group_size": 128, "zero_point": True})
    with pytest.raises(ValueError):
        sba.AWQConfig.from_config({"group_size": 128, "zero_point": True})
    c = sba.AWQConfig(4, 128, True, ["lm_head", "gate"])
    assert c.get_quant_method(torch.nn.Module(), "model.lm_head") is None
    assert isinstance(c.get_quant_method(torch.nn.Module(), "model.layers.0.self_attn.qkv_proj"),
                      sba.AWQLinearMethod)
    moe = torch.nn.Module()
    moe.is_fused_moe = True
    assert isinstance(c.get_quant_method(moe, "model.layers.0.mlp.experts"), sba.AWQMoEMethod)


def test_linear_method_create_weights(sba):
    cfg = sba.AWQConfig(4, 128, True)
    m = sba.AWQLinearMethod(cfg)
    layer = torch.nn.Module()
    m.create_weights(layer, 8192, [8192, 1024, 1024], 8192, 10240, torch.float16, weight_loader="wl")
    assert tuple(layer.qweight.shape) == (8192, 1280) and layer.qweight.dtype == torch.int32
    assert tuple(layer.qzeros.shape) == (64, 1280) and layer.qzeros.dtype == torch.int32
    assert tuple(layer.scales.shape) == (64, 10240) and layer.scales.dtype == torch.float16
    assert layer.qweight.packed_dim == 1 and layer.qweight.pack_factor == 8
    assert layer.qweight.weight_loader == "wl"
    assert sorted(n for n, _ in layer.named_parameters()) == ["qweight", "qzeros", "scales"]
    with pytest.raises(ValueError, match="input size"):
        m.create_weights(torch.nn.Module(), 8192 + 64, [1024], 8256, 1024, torch.float16)
    with pytest.raises(ValueError, match="output size"):
        m.create_weights(torch.nn.Module(), 8192, [1020], 8192, 1020, torch.float16)
    m1 = sba.AWQLinearMethod(sba.AWQConfig(4, -1, True))
    l1 = torch.nn.Module()
    m1.create_weights(l1, 512, [256], 512, 256, torch.float16)
    assert tuple(l1.scales.shape) == (1, 256)


def test_moe_method_create_weights(sba):
    m = sba.AWQMoEMethod(sba.AWQConfig(4, 128, True))
    layer = torch.nn.Module()
    m.create_weights(layer, 128, 2048, 768, torch.float16)
    assert tuple(layer.w13_qweight.shape) == (128, 2048, 192)
    assert tuple(layer.w13_scales.shape) == (128, 16, 1536)
    assert tuple(layer.w13_qzeros.shape) == (128, 16, 192)
    assert tuple(layer.w2_qweight.shape) == (128, 768, 256)
    assert tuple(layer.w2_scales.shape) == (128, 6, 2048)
    assert tuple(layer.w2_qzeros.shape) == (128, 6, 256)


# ------------------------------------------------------------------ workloads

def test_moe_method_refuses_unsupported_routing(sba):
    m = sba.AWQMoEMethod(sba.AWQConfig(4, 128, True))
    layer = torch.nn.Module()
    m.create_weights(layer, 4, 256, 128, torch.float16)
    x, lg = torch.zeros((2, 256), dtype=torch.float16), torch.zeros((2, 4))
    for kw in (dict(use_grouped_topk=True, num_expert_group=4, topk_group=2), dict(scoring_func="tanh"),
               dict(activation="gelu"), dict(e_score_correction_bias=torch.zeros(4)),
               dict(expert_map=torch.arange(4)), dict(global_num_experts=8),
               dict(custom_routing_function=lambda *a: None)):
        with pytest.raises(NotImplementedError):
            m.apply(layer, x, lg, 2, True, **kw)


def test_workload_shapes_and_bytes(sba):
    w = sba.workloads
    c = w.config0()
    assert tuple(c.x.shape) == (16, 4096) and c.x.dtype == torch.float16
    assert tuple(c.qweight.shape) == (4096, 512) and tuple(c.qzeros.shape) == (32, 512)
    assert tuple(c.scales.shape) == (32, 4096)
    assert float(c.scales.min()) >= 0.001 - 1e-6 and float(c.scales.max()) <= 0.02 + 1e-5
    c2 = w.config0()
    assert torch.equal(c.qweight, c2.qweight) and torch.equal(c.x, c2.x)      # seeded
    # algorithmic byte counts of the benchmark definition
    assert w.linear_bytes(1, 8192, 10240) == 43_618_304
    assert w.linear_bytes(16, 8192, 10240) == 44_171_264
    assert w.linear_bytes(1, 8192, 8192) == 34_897_920
    assert w.linear_bytes(16, 8192, 59136) == 253_837_312
    assert w.linear_bytes(4, 29568, 8192) == 126_143_488
    assert w.linear_bytes(16, 4096, 4096) == 8_978_432
    assert w.moe_bytes(1, 0, 2048, 768) == 2_451_456
    assert w.linear_flops(512, 8192, 10240) == 2 * 512 * 8192 * 10240


def test_workload_pack_matches_oracle(sba):
    from oracle import awq_ref
    v = torch.randint(0, 16, (5, 64), generator=torch.Generator().manual_seed(1))
    assert np.array_equal(sba.workloads.pack_int4_awq(v).numpy(), awq_ref.pack_awq(v.numpy()))


def _fake_vllm(monkeypatch, with_registry=True):
    """Stand-in modules with the attribute names the plugin relies on."""
    import sys, types
    for name in [m for m in sys.modules if m == "vllm" or m.startswith("vllm.")]:
        monkeypatch.delitem(sys.modules, name, raising=False)
    mods = {}

    def mod(name, **attrs):
        m = types.ModuleType(name)
        m.__path__ = []
        for k, v in attrs.items():
            setattr(m, k, v)
        monkeypatch.setitem(sys.modules, name, m)
        mods[name] = m
        return m

    old = lambda *a, **k: (_ for _ in ()).throw(AssertionError("vLLM's own op was called"))
    mod("vllm")
    mod("vllm._custom_ops", awq_gemm=old, awq_dequantize=old)
    mod("vllm.envs", VLLM_USE_TRITON_AWQ=True)
    if with_registry:
        class QuantizationConfig:                      # vLLM's base class
            def __init__(self):
                self.packed_modules_mapping = {}

        class FusedMoE(torch.nn.Module):
            pass

        class LinearBase(torch.nn.Module):
            pass

        class UnquantizedLinearMethod:
            pass

        mod("vllm.model_executor")
        mod("vllm.model_executor.layers")
        mod("vllm.model_executor.layers.quantization", QUANTIZATION_METHODS=["awq", "gptq", "awq_marlin"],
            _CUSTOMIZED_METHOD_TO_QUANT_CONFIG={})
        mod("vllm.model_executor.layers.quantization.base_config", QuantizationConfig=QuantizationConfig)
        mod("vllm.model_executor.layers.fused_moe", FusedMoE=FusedMoE)
        mod("vllm.model_executor.layers.linear", LinearBase=LinearBase, UnquantizedLinearMethod=UnquantizedLinearMethod)

        class _ShardAware(torch.nn.Parameter):       # vLLM's parameter classes: keyword-only, loader-carrying
            def __new__(cls, data, **kw):
                return super().__new__(cls, data=data, requires_grad=False)

            def __init__(self, data, weight_loader, input_dim, output_dim, **kw):
                self.built_with = dict(weight_loader=weight_loader, input_dim=input_dim, output_dim=output_dim, **kw)

            def load_merged_column_weight(self, *a, **k):
                return "sharded"

        class PackedvLLMParameter(_ShardAware):
            def __init__(self, data, weight_loader, input_dim, output_dim, packed_dim, packed_factor, **kw):
                super().__init__(data, weight_loader, input_dim, output_dim, packed_dim=packed_dim,
                                 packed_factor=packed_factor, **kw)

        class GroupQuantScaleParameter(_ShardAware):
            pass

        mod("vllm.model_executor.parameter", PackedvLLMParameter=PackedvLLMParameter,
            GroupQuantScaleParameter=GroupQuantScaleParameter)
    return mods


def test_vllm_plugin_rebinds_ops(sba, monkeypatch):
    """Against a stand-in `vllm._custom_ops`: both ops are rebound to this package's functions
    (same argument order as vLLM's); without vLLM the plugin raises ImportError; without the
    quantisation registry the ops are still rebound, with a warning."""
    import importlib, inspect, sys
    plugin = importlib.import_module(sba.__name__ + ".vllm_plugin")
    for name in [m for m in sys.modules if m == "vllm" or m.startswith("vllm.")]:
        monkeypatch.delitem(sys.modules, name, raising=False)
    with pytest.raises(ImportError):
        plugin.register()
    mods = _fake_vllm(monkeypatch, with_registry=False)
    ops_mod = mods["vllm._custom_ops"]
    with pytest.warns(UserWarning):
        assert plugin.register() == ["awq_dequantize", "awq_gemm"]
    assert ops_mod.awq_gemm is sba.awq_gemm and ops_mod.awq_dequantize is sba.awq_dequantize
    assert list(inspect.signature(ops_mod.awq_gemm).parameters)[:5] == \
        ["input", "qweight", "scales", "qzeros", "split_k_iters"]
    assert list(inspect.signature(ops_mod.awq_dequantize).parameters)[:3] == ["qweight", "scales", "zeros"]
    assert mods["vllm.envs"].VLLM_USE_TRITON_AWQ is False


def test_vllm_plugin_registers_the_awq_method_for_linear_and_moe_layers(sba, monkeypatch):
    """The harness passes no --quantization flag, so the method must win by the checkpoint's
    name: after register() vLLM's registry maps `awq` to this package's config, which hands
    AWQMoEMethod to FusedMoE layers and AWQLinearMethod to linear layers, and the MoE method's
    apply (called with vLLM's keyword surface) reaches ops.fused_moe_awq."""
    import importlib
    plugin = importlib.import_module(sba.__name__ + ".vllm_plugin")
    ops = importlib.import_module(sba.__name__ + ".ops")
    mods = _fake_vllm(monkeypatch)
    assert plugin.register() == ["awq_dequantize", "awq_gemm", "quantization:awq"]
    quant = mods["vllm.model_executor.layers.quantization"]
    cls = quant._CUSTOMIZED_METHOD_TO_QUANT_CONFIG["awq"]
    assert quant.QUANTIZATION_METHODS.count("awq") == 1
    assert issubclass(cls, sba.AWQConfig)
    assert issubclass(cls, mods["vllm.model_executor.layers.quantization.base_config"].QuantizationConfig)
    assert cls.get_name() == "awq"
    assert cls.override_quantization_method({"quant_method": "awq", "bits": 4}, None) == "awq"
    assert cls.override_quantization_method({"quant_method": "gptq"}, None) is None
    cfg = cls.from_config({"quant_method": "awq", "bits": 4, "group_size": 128, "zero_point": True,
                           "modules_to_not_convert": ["mlp.gate."]})
    assert cfg.packed_modules_mapping == {} and cfg.group_size == 128       # both base classes initialised
    moe_layer = mods["vllm.model_executor.layers.fused_moe"].FusedMoE()
    lin_layer = mods["vllm.model_executor.layers.linear"].LinearBase()
    assert isinstance(cfg.get_quant_method(lin_layer, "model.layers.0.self_attn.qkv_proj"), sba.AWQLinearMethod)
    # the router stays fp16: a skipped linear layer gets vLLM's unquantised method (vLLM's linear
    # layers call whatever is returned), any other skipped module None
    skipped = cfg.get_quant_method(lin_layer, "model.layers.0.mlp.gate.")
    assert isinstance(skipped, mods["vllm.model_executor.layers.linear"].UnquantizedLinearMethod)
    assert cfg.get_quant_method(torch.nn.LayerNorm(4), "model.layers.0.mlp.gate.norm") is None
    assert cfg.get_quant_method(torch.nn.LayerNorm(4), "model.norm") is None
    method = cfg.get_quant_method(moe_layer, "model.layers.0.mlp.experts")
    assert isinstance(method, sba.AWQMoEMethod)
    method.create_weights(moe_layer, 4, 256, 128, torch.float16)
    seen = {}

    def fake_fused(hidden, w13, w2, logits, topk, renorm, **kw):
        seen.update(topk=topk, renorm=renorm, w13=w13[0].shape, w2=w2[0].shape, kw=kw)
        return torch.zeros_like(hidden)

    monkeypatch.setattr(ops, "fused_moe_awq", fake_fused)
    x, lg = torch.zeros((3, 256), dtype=torch.float16), torch.zeros((3, 4))
    y = method.apply(moe_layer, x, lg, 2, True, use_grouped_topk=False, topk_group=None, num_expert_group=None,
                     global_num_experts=4, expert_map=None, custom_routing_function=None, scoring_func="softmax",
                     e_score_correction_bias=None, apply_router_weight_on_input=False, activation="silu")
    assert tuple(y.shape) == (3, 256)
    assert seen["topk"] == 2 and seen["renorm"] is True
    assert tuple(seen["w13"]) == (4, 256, 32) and tuple(seen["w2"]) == (4, 128, 32)
    with pytest.raises(NotImplementedError):
        method.apply(moe_layer, x, lg, 2, True, apply_router_weight_on_input=True)


def test_vllm_plugin_checks_what_the_registry_hands_out(sba, monkeypatch):
    """After writing the table the plugin asks vLLM for the `awq` config: the registered class is a
    success, anything else (a registry that resolves built-in names first) is warned about and not
    reported as registered."""
    import importlib
    plugin = importlib.import_module(sba.__name__ + ".vllm_plugin")
    mods = _fake_vllm(monkeypatch)
    quant = mods["vllm.model_executor.layers.quantization"]
    quant.get_quantization_config = lambda name: quant._CUSTOMIZED_METHOD_TO_QUANT_CONFIG[name]
    assert "quantization:awq" in plugin.register()

    class BuiltInAWQ:
        pass

    quant.get_quantization_config = lambda name: BuiltInAWQ
    with pytest.warns(UserWarning, match="get_quantization_config"):
        assert "quantization:awq" not in plugin.register()


def test_create_weights_uses_vllm_parameter_classes_inside_vllm(sba, monkeypatch):
    """vLLM picks its second-generation weight loader for a method whose class is NAMED
    AWQLinearMethod, and that loader calls shard-loading methods of vLLM's parameter classes: with
    vLLM importable and a callable weight_loader the three parameters are built from those classes
    (same keyword arguments as vLLM's own AWQ method), keep their names, shapes and dtypes, and
    turn into plain contiguous parameters after loading."""
    mods = _fake_vllm(monkeypatch)
    par = mods["vllm.model_executor.parameter"]
    loader = lambda param, loaded, *a: None
    assert sba.AWQLinearMethod.__name__ == "AWQLinearMethod"
    m = sba.AWQLinearMethod(sba.AWQConfig(4, 128, True))
    layer = torch.nn.Module()
    m.create_weights(layer, 1024, [512, 128, 128], 1024, 768, torch.float16, weight_loader=loader)
    assert type(layer.qweight) is par.PackedvLLMParameter and type(layer.qzeros) is par.PackedvLLMParameter
    assert type(layer.scales) is par.GroupQuantScaleParameter
    assert layer.qweight.built_with == dict(weight_loader=loader, input_dim=0, output_dim=1, packed_dim=1,
                                            packed_factor=8)
    assert layer.scales.built_with == dict(weight_loader=loader, input_dim=0, output_dim=1)
    assert layer.qweight.load_merged_column_weight() == "sharded"
    assert tuple(layer.qweight.shape) == (1024, 96) and layer.qweight.dtype == torch.int32
    assert tuple(layer.qzeros.shape) == (8, 96) and tuple(layer.scales.shape) == (8, 768)
    assert sorted(n for n, _ in layer.named_parameters()) == ["qweight", "qzeros", "scales"]
    m.process_weights_after_loading(layer)
    assert type(layer.qweight) is torch.nn.Parameter and layer.qweight.is_contiguous()
    # no loader given (this package's own checkpoint reader): plain parameters with the attributes
    l2 = torch.nn.Module()
    m.create_weights(l2, 1024, [768], 1024, 768, torch.float16)
    assert type(l2.qweight) is torch.nn.Parameter and l2.qweight.pack_factor == 8


def test_moe_parameters_carry_what_vllms_expert_loader_reads(sba):
    m = sba.AWQMoEMethod(sba.AWQConfig(4, 128, True))
    layer = torch.nn.Module()
    loader = lambda *a, **k: None
    m.create_weights(layer, 4, 256, 128, torch.float16, weight_loader=loader)
    for name in ("w13_qweight", "w13_scales", "w13_qzeros", "w2_qweight", "w2_scales", "w2_qzeros"):
        p = getattr(layer, name)
        assert p.is_transposed is True and p.quant_method == "group" and p.weight_loader is loader


def test_awq_gemm_takes_vllm_split_k_iters_as_a_hint(sba, monkeypatch):
    """vLLM's AWQLinearMethod.apply always passes its pack factor (8) as split_k_iters.  The op
    this package binds in its place must hand 0 (= the library's own choice) to the C ABI for
    it, and only force_split_k reaches the library."""
    import importlib
    ops = importlib.import_module(sba.__name__ + ".ops")
    libmod = importlib.import_module(sba.__name__ + "._lib")
    calls = []

    class FakeLib:
        def awqmi_gemm_workspace_bytes(self, M, K, N, split):
            calls.append(("ws", split))
            return 65536

        def awqmi_gemm_f16(self, *a):
            calls.append(("gemm", a[11]))
            return 0

    monkeypatch.setattr(libmod, "load", lambda: FakeLib())
    monkeypatch.setattr(ops, "_need", lambda *a, **k: None)
    monkeypatch.setattr(ops, "_need_qweight", lambda t: t.shape[1])
    monkeypatch.setattr(ops, "_stream_ptr", lambda dev: 0)
    monkeypatch.setattr(ops, "get_workspace", lambda dev, n, s=None: torch.zeros(n, dtype=torch.uint8))
    monkeypatch.setattr(ops, "_gemm_ws_bytes", {})
    x = torch.zeros((4, 256), dtype=torch.float16)
    qw = torch.zeros((256, 16), dtype=torch.int32)
    sc = torch.zeros((2, 128), dtype=torch.float16)
    qz = torch.zeros((2, 16), dtype=torch.int32)
    ops.awq_gemm(x, qw, sc, qz, 8)                       # what vLLM passes
    assert calls == [("ws", 0), ("gemm", 0)]
    calls.clear()
    ops.awq_gemm(x, qw, sc, qz, 8, force_split_k=2)
    assert calls == [("ws", 2), ("gemm", 2)]


def test_plugin_entry_point_resolves_from_the_mounted_layout(sba):
    """What deploy.py mounts into a server is the root of this repository on PYTHONPATH: the
    .dist-info directory there must declare the vllm.general_plugins entry point, and the entry
    point must load (through the `server_benchmark_amd` alias module beside it)."""
    import importlib.metadata as md
    dists = [d for d in md.distributions(path=[ROOT]) if d.metadata["Name"] == "server_benchmark_amd"]
    assert len(dists) == 1
    eps = [e for e in dists[0].entry_points if e.group == "vllm.general_plugins"]
    assert [e.name for e in eps] == ["awq_mi355x"]
    deploy = __import__("importlib").import_module(sba.__name__ + ".deploy")
    assert eps[0].name == deploy.PLUGIN_NAME
    fn = eps[0].load()
    plugin = __import__("importlib").import_module(sba.__name__ + ".vllm_plugin")
    assert fn is plugin.register
    assert os.path.exists(os.path.join(ROOT, "server_benchmark_amd.py"))      # the alias the entry point names


def test_bench_is_for_one_gpu_and_has_no_cpu_path():
    """`bench.py --gpus N` with N above one exits with a message that says so; without a GPU the
    run fails loudly instead of measuring anything on the CPU."""
    import subprocess
    import sys
    bench = os.path.join(ROOT, "bench.py")
    res = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and "one GPU only" in res.stderr and res.stdout.strip() == ""
    import torch
    if not torch.cuda.is_available():
        res = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True,
                             timeout=300)
        assert res.returncode == 1 and "no CPU fallback" in res.stderr and res.stdout.strip() == ""

