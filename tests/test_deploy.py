"""ROCm deployment description against a compose file the harness recorded
(tests/golden/compose/*.yml is the "Docker Compose Configuration" block of one of its result
files, 4 instances x 1 GPU behind nginx): everything that does not depend on the GPU vendor
must come out the same; the GPU plumbing must be ROCm's."""
import pathlib
from importlib import import_module

import pytest
import yaml

GOLD = pathlib.Path(__file__).parent / "golden" / "compose" / "rtx5090_x_4_qwen3_coder_30b_awq.yml"
MODEL = "QuantTrio/Qwen3-Coder-30B-A3B-Instruct-AWQ"


@pytest.fixture(scope="module")
def deploy(sba):
    return import_module(sba.__name__ + ".deploy")


@pytest.fixture(scope="module")
def stack(deploy):
    return deploy.compose(4, 1, 1, "vllm_benchmark_container", f"/hf_models/{MODEL}", MODEL, "/hf_models",
                          nginx_conf_path="/home/riftuser/server-benchmark/nginx.vllm.conf",
                          extra_args="--max-model-len 8192", total_gpus=4)


def test_vendor_independent_parts_match_the_recorded_stack(deploy, stack):
    want = yaml.safe_load(GOLD.read_text())["services"]
    got = yaml.safe_load(deploy.to_yaml(stack))["services"]          # through the YAML text
    assert list(got) == list(want)
    for i in range(4):
        g, w = got[f"vllm_{i}"], want[f"vllm_{i}"]
        for key in ("container_name", "ports", "shm_size", "ipc", "healthcheck"):
            assert g[key] == w[key], key
        assert g["command"].split() == w["command"].split()
        assert g["volumes"][0] == w["volumes"][0]
        assert g["environment"][0] == w["environment"][0]
    assert got["nginx"] == want["nginx"]
    for key in ("container_name", "volumes", "entrypoint", "command", "profiles"):
        assert got["benchmark"][key] == want["benchmark"][key]


def test_gpu_plumbing_is_rocm(deploy, stack):
    for i in range(4):
        s = stack["services"][f"vllm_{i}"]
        assert s["devices"] == ["/dev/kfd:/dev/kfd", "/dev/dri:/dev/dri"] and s["group_add"] == ["video"]
        assert f"HIP_VISIBLE_DEVICES={i}" in s["environment"]
        assert "deploy" not in s and not any("CUDA" in e or "NVIDIA" in e for e in s["environment"])
    one = deploy.compose(1, 8, 1, "c", "/m", "m", "/hf", total_gpus=8, library_dir="/srv/awq")
    s = one["services"]["vllm_0"]
    assert not any(e.startswith("HIP_VISIBLE_DEVICES") for e in s["environment"])      # sees every GPU
    assert "/srv/awq:/opt/awq_mi355x:ro" in s["volumes"] and "VLLM_USE_TRITON_AWQ=0" in s["environment"]
    assert "nginx" not in one["services"]
    two = deploy.compose(2, 2, 2, "c", "/m", "m", "/hf", total_gpus=8)
    assert "HIP_VISIBLE_DEVICES=4,5,6,7" in two["services"]["vllm_1"]["environment"]
    with pytest.raises(ValueError):
        deploy.compose(3, 4, 1, "c", "/m", "m", "/hf", total_gpus=8)


REFERENCE_RESULTS = pathlib.Path("/root/reference/results")


def _recorded_compose(text):
    """The YAML of the "Docker Compose Configuration" block of a benchmark log, or None."""
    head = "Docker Compose Configuration"
    if head not in text:
        return None
    body = text.split(head, 1)[1].split("\n", 1)[1]
    lines = []
    for line in body.splitlines():
        if line.startswith("====") or line.startswith("----"):
            break
        lines.append(line)
    return yaml.safe_load("\n".join(lines))


@pytest.mark.skipif(not REFERENCE_RESULTS.is_dir(), reason="the harness's recorded results are not on this machine")
def test_every_recorded_stack(deploy):
    """Every compose block the harness recorded, regenerated from its own parameters (instance
    count, parallel sizes, model, extra arguments read off the block): same services, same
    commands, ports, health checks, nginx and benchmark services, and each instance gets the GPU
    indexes the recorded block reserved for it -- as HIP_VISIBLE_DEVICES instead of a
    device reservation."""
    files = sorted(REFERENCE_RESULTS.glob("*/*_vllm_benchmark.txt"))
    checked = 0
    for f in files:
        doc = _recorded_compose(f.read_text(errors="replace"))
        if not doc:
            continue
        want = doc["services"]
        n = sum(1 for k in want if k.startswith("vllm_"))
        cmd = want["vllm_0"]["command"].split()
        if "--pipeline-parallel-size" not in cmd:
            continue          # a block written by an earlier version of the generator
        tp = int(cmd[cmd.index("--tensor-parallel-size") + 1])
        pp = int(cmd[cmd.index("--pipeline-parallel-size") + 1])
        model_path = cmd[cmd.index("--model") + 1]
        k = cmd.index("--served-model-name")
        model_name, extra = cmd[k + 1], " ".join(cmd[k + 2:])
        name = want["vllm_0"]["container_name"].rsplit("_", 1)[0]
        hf_dir = want["vllm_0"]["volumes"][0].split(":")[0]
        conf = want["nginx"]["volumes"][0].split(":")[0] if "nginx" in want else None
        got = yaml.safe_load(deploy.to_yaml(deploy.compose(n, tp, pp, name, model_path, model_name, hf_dir,
                                                           nginx_conf_path=conf, extra_args=extra)))["services"]
        assert list(got) == list(want), f.name
        for i in range(n):
            g, w = got[f"vllm_{i}"], want[f"vllm_{i}"]
            for key in ("container_name", "ports", "shm_size", "ipc", "healthcheck"):
                assert g[key] == w[key], (f.name, key)
            assert g["command"].split() == w["command"].split(), f.name
            ids = w["deploy"]["resources"]["reservations"]["devices"][0]["device_ids"]
            assert f"HIP_VISIBLE_DEVICES={','.join(str(x) for x in ids)}" in g["environment"], f.name
        if "nginx" in want:
            assert got["nginx"] == want["nginx"], f.name
        for key in ("container_name", "volumes", "entrypoint", "command", "profiles"):
            assert got["benchmark"][key] == want["benchmark"][key], (f.name, key)
        checked += 1
    print(f"[deploy] {checked} recorded stacks regenerated")
    assert checked >= 10


def test_gpu_count_and_nginx_conf(deploy):
    text = "\n".join(["Agent 1", "  Device Type:             CPU", "Agent 2", "  Device Type:             GPU",
                      "  Compute Unit:            256", "Agent 3", "  Device Type:             GPU"])
    assert deploy.count_rocm_gpus(text) == 2 and deploy.count_rocm_gpus("") == 0
    conf = deploy.nginx_conf(3)
    assert conf.count("server vllm_") == 3 and "least_conn;" in conf and "listen 8080;" in conf
    assert "proxy_buffering off;" in conf and conf.count("{") == conf.count("}")


def test_cli_writes_the_recorded_stack(deploy, tmp_path, monkeypatch):
    """The command line the harness's step script uses for its own generator (reference
    benchmarks/3_vllm_benchmark.sh:46-63, flags of utils/generate_compose.py:261-332), pointed
    at this file: the files it writes must carry the recorded stack's vendor-independent parts
    and nginx.conf, and the reference's messages."""
    out, conf = tmp_path / "docker-compose.vllm.yml", tmp_path / "nginx.vllm.conf"
    monkeypatch.setattr(deploy, "total_rocm_gpus", lambda: 4)
    argv = ["--num-instances", "4", "--tensor-parallel-size", "1", "--pipeline-parallel-size", "1",
            "--container-name", "vllm_benchmark_container", "--model-path", f"/hf_models/{MODEL}",
            "--model-name", MODEL, "--hf-directory", "/hf_models", "--hf-token", "",
            "--extra-args", "--max-model-len 8192", "--output", str(out), "--nginx-conf-output", str(conf)]
    assert deploy.main(argv) == 0
    want = yaml.safe_load(GOLD.read_text())["services"]
    got = yaml.safe_load(out.read_text())["services"]
    assert list(got) == list(want)
    for i in range(4):
        g, w = got[f"vllm_{i}"], want[f"vllm_{i}"]
        for key in ("container_name", "ports", "shm_size", "ipc", "healthcheck"):
            assert g[key] == w[key], key
        assert g["command"].split() == w["command"].split()
        assert f"HIP_VISIBLE_DEVICES={i}" in g["environment"]
    assert got["nginx"]["volumes"] == [f"{conf}:/etc/nginx/nginx.conf:ro"]       # absolute path, as docker wants it
    assert got["nginx"]["depends_on"] == want["nginx"]["depends_on"]
    assert conf.read_text() == deploy.nginx_conf(4)
    # several instances without a place for nginx.conf: the reference's error, exit status 1
    assert deploy.main(argv[:-2]) == 1
    # one instance that takes every GPU of the host sees all devices; with the library mounted the
    # server gets the plugin's path
    one = tmp_path / "one.yml"
    monkeypatch.setattr(deploy, "total_rocm_gpus", lambda: 8)
    assert deploy.main(["--num-instances", "1", "--tensor-parallel-size", "8", "--container-name", "c",
                        "--model-path", "/m", "--model-name", "m", "--hf-directory", "/hf", "-o", str(one),
                        "--library-dir", "/srv/awq"]) == 0
    svc = yaml.safe_load(one.read_text())["services"]["vllm_0"]
    assert not any(e.startswith("HIP_VISIBLE_DEVICES") for e in svc["environment"])
    assert "/srv/awq:/opt/awq_mi355x:ro" in svc["volumes"] and "PYTHONPATH=/opt/awq_mi355x" in svc["environment"]
    with pytest.raises(SystemExit):
        deploy.main(["--num-instances", "1"])


def test_gpu_count_runs_rocminfo_and_system_info_section(deploy):
    import subprocess
    text = "\n".join(["Agent 1", "  Device Type:             CPU", "Agent 2", "  Device Type:             GPU",
                      "Agent 3", "  Device Type:             GPU"])
    calls = []

    def runner(cmd, **kw):
        calls.append(cmd)
        assert kw.get("check") and kw.get("capture_output") and kw.get("text")
        if cmd[0] == "rocminfo":
            return subprocess.CompletedProcess(cmd, 0, stdout=text, stderr="")
        if cmd == ["rocm-smi"]:
            return subprocess.CompletedProcess(cmd, 0, stdout="GPU  Temp  Power\n0    35c   140W\n", stderr="")
        raise subprocess.CalledProcessError(2, cmd)

    def absent(cmd, **kw):
        raise FileNotFoundError(cmd[0])

    assert deploy.total_rocm_gpus(runner) == 2 and calls == [["rocminfo"]]
    assert deploy.total_rocm_gpus(absent) == 0                 # no tool: 0 GPUs, as the harness counts
    sec = deploy.system_info_gpu_section(runner)
    assert sec.startswith("=== GPU INFORMATION ===\n")
    assert "=== ROCM-SMI FULL OUTPUT ===\nGPU  Temp  Power" in sec and "=== ROCMINFO (2 GPU agents) ===" in sec
    assert deploy.system_info_gpu_section(absent) == "=== GPU INFORMATION ===\nNo GPU information available\n"
