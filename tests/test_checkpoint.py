"""AWQ checkpoint reader on small checkpoints written here with safetensors: tensors come back
bit for bit, merged projections and expert stacks land where the layer methods expect them,
and malformed folders are refused with a reason."""
import json
from importlib import import_module

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from oracle import awq_ref


@pytest.fixture(scope="module")
def ck(sba):
    return import_module(sba.__name__ + ".checkpoint")


def _triple(sba, K, N, G, seed):
    gen = torch.Generator().manual_seed(seed)
    return sba.workloads.make_awq_weights(K, N, G, gen)      # (qweight, scales, qzeros)


def _write(tmp_path, tensors, quant=None, where="config.json", shards=1):
    quant = quant if quant is not None else {"quant_method": "awq", "bits": 4, "group_size": 128,
                                             "zero_point": True, "version": "gemm"}
    if where == "config.json":
        (tmp_path / "config.json").write_text(json.dumps({"model_type": "tiny", "quantization_config": quant}))
    else:
        (tmp_path / "config.json").write_text(json.dumps({"model_type": "tiny"}))
        (tmp_path / where).write_text(json.dumps(quant))
    names = sorted(tensors)
    if shards == 1:
        save_file({n: tensors[n] for n in names}, str(tmp_path / "model.safetensors"))
    else:
        wm = {}
        for i in range(shards):
            part = names[i::shards]
            fn = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
            save_file({n: tensors[n] for n in part}, str(tmp_path / fn))
            wm.update({n: fn for n in part})
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": wm}))
    return tmp_path


def _named(prefix, triple):
    qw, sc, qz = triple
    return {f"{prefix}.qweight": qw, f"{prefix}.scales": sc, f"{prefix}.qzeros": qz}


def test_config_sources(sba, ck, tmp_path):
    t = _named("m.q", _triple(sba, 256, 64, 128, 1))
    a = tmp_path / "a"; a.mkdir()
    c = ck.read_awq_config(_write(a, t))
    assert (c.weight_bits, c.group_size, c.zero_point) == (4, 128, True)
    b = tmp_path / "b"; b.mkdir()
    c = ck.read_awq_config(_write(b, t, quant={"w_bit": 4, "q_group_size": 64, "zero_point": True},
                                  where="quant_config.json"))
    assert c.group_size == 64
    for bad, why in (({"quant_method": "gptq", "bits": 4, "group_size": 128, "zero_point": True}, "gptq"),
                     ({"quant_method": "awq", "bits": 4, "group_size": 128, "zero_point": True, "version": "gemv"}, "gemv"),
                     ({"quant_method": "awq", "bits": 8, "group_size": 128, "zero_point": True}, "4-bit")):
        d = tmp_path / why; d.mkdir()
        with pytest.raises(ck.CheckpointError, match=why):
            ck.read_awq_config(_write(d, t, quant=bad))
    e = tmp_path / "none"; e.mkdir()
    (e / "config.json").write_text("{}")
    with pytest.raises(ck.CheckpointError):
        ck.read_awq_config(e)


def test_linear_round_trip_and_merge(sba, ck, tmp_path):
    q, k, v = (_triple(sba, 256, n, 128, s) for n, s in ((128, 2), (64, 3), (64, 4)))
    tensors = {**_named("l.q_proj", q), **_named("l.k_proj", k), **_named("l.v_proj", v),
               "l.norm.weight": torch.ones(256, dtype=torch.float16)}
    cp = ck.AWQCheckpoint(_write(tmp_path, tensors, shards=2))
    assert cp.linear_prefixes() == ["l.k_proj", "l.q_proj", "l.v_proj"]
    for got, want in zip(cp.read_linear("l.q_proj"), q):
        assert torch.equal(got, want)
    method = sba.AWQLinearMethod(cp.config)
    layer = torch.nn.Module()
    method.create_weights(layer, 256, [128, 64, 64], 256, 256, torch.float16)
    cp.load_linear(layer, ["l.q_proj", "l.k_proj", "l.v_proj"])
    # the merged layer dequantises to the three parts side by side
    W = awq_ref.dequantize(layer.qweight.numpy(), layer.scales.numpy(), layer.qzeros.numpy(), 128)
    parts = [awq_ref.dequantize(t[0].numpy(), t[1].numpy(), t[2].numpy(), 128) for t in (q, k, v)]
    assert np.array_equal(W.view(np.uint16), np.concatenate(parts, axis=1).view(np.uint16))
    wrong = torch.nn.Module()
    method.create_weights(wrong, 256, [128], 256, 128, torch.float16)
    with pytest.raises(ck.CheckpointError, match="layer shape"):
        cp.load_linear(wrong, ["l.q_proj", "l.k_proj"])
    with pytest.raises(ck.CheckpointError, match="not found"):
        cp.read_linear("l.o_proj")


def test_expert_stacks(sba, ck, tmp_path):
    E, H, I = 3, 256, 128
    tensors, trip = {}, {}
    for e in range(E):
        for j, (name, K, N) in enumerate((("gate_proj", H, I), ("up_proj", H, I), ("down_proj", I, H))):
            trip[e, name] = _triple(sba, K, N, 128, 10 * e + j)
            tensors.update(_named(f"mlp.experts.{e}.{name}", trip[e, name]))
    cp = ck.AWQCheckpoint(_write(tmp_path, tensors))
    method = sba.AWQMoEMethod(cp.config)
    layer = torch.nn.Module()
    method.create_weights(layer, E, H, I, torch.float16)
    cp.load_experts(layer, "mlp.experts", E)
    for e in range(E):
        assert torch.equal(layer.w13_qweight[e][:, : I // 8], trip[e, "gate_proj"][0])
        assert torch.equal(layer.w13_qweight[e][:, I // 8:], trip[e, "up_proj"][0])
        assert torch.equal(layer.w13_scales[e][:, I:], trip[e, "up_proj"][1])
        assert torch.equal(layer.w2_qzeros[e], trip[e, "down_proj"][2])


def test_malformed_tensors_are_refused(sba, ck, tmp_path):
    qw, sc, qz = _triple(sba, 256, 64, 128, 5)
    cases = {
        "dtype": _named("x", (qw, sc.float(), qz)),
        "zshape": _named("x", (qw, sc, qz[:1])),
        "sshape": _named("x", (qw, sc[:, :32].contiguous(), qz)),
        "group": _named("x", (qw[:200].contiguous(), sc, qz)),
    }
    for name, tensors in cases.items():
        d = tmp_path / name; d.mkdir()
        cp = ck.AWQCheckpoint(_write(d, tensors))
        with pytest.raises(ck.CheckpointError):
            cp.read_linear("x")
    empty = tmp_path / "empty"; empty.mkdir()
    (empty / "config.json").write_text(json.dumps({"quantization_config": {"bits": 4, "group_size": 128, "zero_point": True}}))
    with pytest.raises(ck.CheckpointError, match="safetensors"):
        ck.AWQCheckpoint(empty)


@pytest.mark.gpu
def test_checkpoint_to_gpu_layer_apply(sba, ck, gpu, tmp_path):
    """Folder -> layer parameters on the device -> AWQLinearMethod.apply, against the oracle."""
    gate, up = _triple(sba, 512, 256, 128, 21), _triple(sba, 512, 256, 128, 22)
    cp = ck.AWQCheckpoint(_write(tmp_path, {**_named("mlp.gate_proj", gate), **_named("mlp.up_proj", up)}))
    method = sba.AWQLinearMethod(cp.config)
    layer = torch.nn.Module()
    method.create_weights(layer, 512, [256, 256], 512, 512, torch.float16, device=gpu)
    cp.load_linear(layer, ["mlp.gate_proj", "mlp.up_proj"])
    method.process_weights_after_loading(layer)
    x = torch.randn((5, 512), generator=torch.Generator().manual_seed(3)).half()
    y = method.apply(layer, x.to(gpu)).cpu().numpy()
    ref = np.concatenate([awq_ref.gemm_wide(x.numpy(), t[0].numpy(), t[1].numpy(), t[2].numpy(), 128)
                          for t in (gate, up)], axis=1)
    assert awq_ref.rel_frobenius(y, ref) <= 2e-3
