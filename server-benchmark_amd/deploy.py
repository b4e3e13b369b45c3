"""docker-compose description of the serving stack for an MI355X host.

ROCm counterpart of the deployment the harness generates (reference
utils/generate_compose.py:46-100 vLLM service, :103-118 nginx, :121-143 benchmark client,
:146-190 nginx.conf, :12-43 GPU count): the same services, ports, volumes, server command
and health check, with the GPU plumbing of a ROCm container (/dev/kfd + /dev/dri, group
`video`, `HIP_VISIBLE_DEVICES`) in place of the NVIDIA runtime reservation, and with this
library mounted into the server so that its AWQ layers run on it.  The stack is built as
plain data and serialised with yaml.safe_dump; nothing here talks to docker.

Command line (same flags as the harness's generator, reference utils/generate_compose.py:261-332,
so that its step script benchmarks/3_vllm_benchmark.sh:46-81 can call this file in its place):

    python deploy.py --num-instances N --tensor-parallel-size T [--pipeline-parallel-size P]
        --container-name C --model-path M --model-name NAME --hf-directory D [--hf-token TOK]
        [--extra-args "..."] --output docker-compose.yml [--nginx-conf-output nginx.conf]
        [--library-dir DIR] [--image IMAGE]

    python deploy.py --system-info     # the ROCm lines of the system-information step

The GPU count comes from running `rocminfo` (an absent or failing tool counts as 0 GPUs, as
the harness does for its own tool at reference utils/generate_compose.py:40-42).
"""
from __future__ import annotations

import argparse
import os
import re
import subprocess
import sys
from typing import Optional

import yaml

ROCM_VLLM_IMAGE = "rocm/vllm:latest"
PLUGIN_MOUNT = "/opt/awq_mi355x"
PLUGIN_NAME = "awq_mi355x"          # entry-point name in the .dist-info next to the package
HEALTHCHECK = ("curl -f http://localhost:8000/health && "
               "curl -f http://localhost:8000/v1/models | grep -q 'object.*list'")


def count_rocm_gpus(rocminfo_text: str) -> int:
    """GPU agents in `rocminfo` output (agents whose Device Type is GPU)."""
    return len(re.findall(r"^\s*Device Type:\s+GPU\s*$", rocminfo_text, flags=re.M))


def total_rocm_gpus(runner=subprocess.run) -> int:
    """GPU agents of this host as `rocminfo` lists them; 0 when the tool is absent or fails
    (counterpart of reference utils/generate_compose.py:12-43, which asks nvidia-smi)."""
    try:
        res = runner(["rocminfo"], capture_output=True, text=True, check=True)
    except (subprocess.CalledProcessError, FileNotFoundError, PermissionError):
        return 0
    return count_rocm_gpus(res.stdout)


def system_info_gpu_section(runner=subprocess.run) -> str:
    """The "GPU INFORMATION" part of the system-information step for a ROCm host (counterpart of
    reference benchmarks/1_system_info.sh:68-82, which prints a csv query and the full output of
    its vendor tool): the product / memory / driver query of rocm-smi, its full table, and the
    agent list of rocminfo; tools that are absent are named as such, as the step does."""
    def run(cmd):
        try:
            return runner(cmd, capture_output=True, text=True, check=True).stdout.rstrip("\n")
        except (subprocess.CalledProcessError, FileNotFoundError, PermissionError):
            return None
    lines = ["=== GPU INFORMATION ==="]
    q = run(["rocm-smi", "--showproductname", "--showmeminfo", "vram", "--showdriverversion", "--csv"])
    full = run(["rocm-smi"])
    agents = run(["rocminfo"])
    if q is None and full is None and agents is None:
        lines.append("No GPU information available")
        return "\n".join(lines) + "\n"
    if q is not None:
        lines += [q, ""]
    if full is not None:
        lines += ["=== ROCM-SMI FULL OUTPUT ===", full, ""]
    if agents is not None:
        lines += [f"=== ROCMINFO ({count_rocm_gpus(agents)} GPU agents) ===", agents]
    return "\n".join(lines) + "\n"


def gpu_ids(instance_id: int, gpus_per_instance: int) -> list:
    start = instance_id * gpus_per_instance
    return list(range(start, start + gpus_per_instance))


def _rocm_plumbing(visible: Optional[list]) -> dict:
    d = {
        "devices": ["/dev/kfd:/dev/kfd", "/dev/dri:/dev/dri"],
        "group_add": ["video"],
        "cap_add": ["SYS_PTRACE"],
        "security_opt": ["seccomp=unconfined"],
    }
    if visible is not None:
        d["_visible"] = ",".join(str(g) for g in visible)
    return d


def vllm_service(instance_id: int, visible: Optional[list], container_name: str, tensor_parallel_size: int,
                 pipeline_parallel_size: int, model_path: str, model_name: str, hf_directory: str,
                 hf_token: str = "", extra_args: str = "", library_dir: Optional[str] = None,
                 image: str = ROCM_VLLM_IMAGE) -> dict:
    """One server instance.  visible = GPU indices of this instance, None = all GPUs."""
    plumbing = _rocm_plumbing(visible)
    env = [f"HUGGING_FACE_HUB_TOKEN={hf_token}", f"HF_HOME={hf_directory}"]
    if "_visible" in plumbing:
        env.append(f"HIP_VISIBLE_DEVICES={plumbing.pop('_visible')}")
    volumes = [f"{hf_directory}:{hf_directory}"]
    if library_dir:
        # The root of this repository (package directory with libawq_mi355x.so inside, the
        # `server_benchmark_amd` import alias and the .dist-info directory that declares the
        # vllm.general_plugins entry point) on the server's Python path: vLLM finds the entry
        # point through importlib.metadata and calls vllm_plugin.register() in every worker.
        volumes.append(f"{library_dir}:{PLUGIN_MOUNT}:ro")
        env.append(f"PYTHONPATH={PLUGIN_MOUNT}")
        env.append("VLLM_USE_TRITON_AWQ=0")
    command = ["--trust-remote-code", "--gpu-memory-utilization=0.9", "--host 0.0.0.0", "--port 8000",
               f"--tensor-parallel-size {tensor_parallel_size}",
               f"--pipeline-parallel-size {pipeline_parallel_size}",
               f"--model {model_path}", f"--served-model-name {model_name}"]
    if extra_args.strip():
        command.append(extra_args.strip())
    svc = {
        "image": image,
        "container_name": f"{container_name}_{instance_id}",
        **plumbing,
        "volumes": volumes,
        "environment": env,
        "ports": [f"{8000 + instance_id}:8000"],
        "shm_size": "16gb",
        "ipc": "host",
        "command": " ".join(command),
        "healthcheck": {"test": ["CMD", "bash", "-c", HEALTHCHECK], "interval": "10s", "timeout": "10s",
                        "retries": 180, "start_period": "600s"},
    }
    return svc


def nginx_service(num_instances: int, nginx_conf_path: str) -> dict:
    return {"image": "nginx:alpine", "container_name": "nginx_lb", "ports": ["8080:8080"],
            "volumes": [f"{nginx_conf_path}:/etc/nginx/nginx.conf:ro"],
            "depends_on": [f"vllm_{i}" for i in range(num_instances)]}


def benchmark_service(hf_directory: str, hf_token: str = "", image: str = ROCM_VLLM_IMAGE) -> dict:
    """The client container `vllm bench serve` is exec'ed in; it needs no GPU."""
    return {"image": image, "container_name": "vllm_benchmark_client",
            "volumes": [f"{hf_directory}:{hf_directory}"],
            "environment": [f"HUGGING_FACE_HUB_TOKEN={hf_token}", f"HF_HOME={hf_directory}",
                            'HIP_VISIBLE_DEVICES=""'],
            "entrypoint": ["/bin/bash", "-c"], "command": ["sleep infinity"], "profiles": ["tools"]}


def compose(num_instances: int, tensor_parallel_size: int, pipeline_parallel_size: int, container_name: str,
            model_path: str, model_name: str, hf_directory: str, hf_token: str = "",
            nginx_conf_path: Optional[str] = None, extra_args: str = "", total_gpus: int = 0,
            library_dir: Optional[str] = None, image: str = ROCM_VLLM_IMAGE) -> dict:
    """The whole stack.  One instance that takes every GPU of the host (total_gpus, from
    count_rocm_gpus) sees all devices; otherwise instance i sees GPUs
    [i * tp * pp, (i + 1) * tp * pp).  nginx is added for more than one instance."""
    per = tensor_parallel_size * pipeline_parallel_size
    if num_instances < 1 or per < 1:
        raise ValueError("num_instances and tensor_parallel_size * pipeline_parallel_size must be >= 1")
    if total_gpus and num_instances * per > total_gpus:
        raise ValueError(f"{num_instances} instances x {per} GPUs exceed the host's {total_gpus} GPUs")
    take_all = num_instances == 1 and total_gpus > 0 and per == total_gpus
    services = {}
    for i in range(num_instances):
        services[f"vllm_{i}"] = vllm_service(i, None if take_all else gpu_ids(i, per), container_name,
                                             tensor_parallel_size, pipeline_parallel_size, model_path,
                                             model_name, hf_directory, hf_token, extra_args, library_dir, image)
    if num_instances > 1 and nginx_conf_path:
        services["nginx"] = nginx_service(num_instances, nginx_conf_path)
    services["benchmark"] = benchmark_service(hf_directory, hf_token, image)
    return {"services": services}


def to_yaml(stack: dict) -> str:
    return yaml.safe_dump(stack, sort_keys=False, default_flow_style=False, width=1000)


def nginx_conf(num_instances: int) -> str:
    """Least-connections load balancer on :8080 over the instances, long timeouts, no buffering
    (streaming responses)."""
    servers = "".join(f"        server vllm_{i}:8000;\n" for i in range(num_instances))
    return ("worker_processes auto;\n\nevents {\n    worker_connections 4096;\n}\n\nhttp {\n"
            "    upstream vllm_backend {\n        least_conn;\n" + servers + "    }\n\n"
            "    server {\n        listen 8080;\n\n        location / {\n"
            "            proxy_pass http://vllm_backend;\n            proxy_http_version 1.1;\n"
            "            proxy_set_header Connection \"\";\n            proxy_set_header Host $host;\n"
            "            proxy_set_header X-Real-IP $remote_addr;\n"
            "            proxy_set_header X-Forwarded-For $proxy_add_x_forwarded_for;\n"
            "            proxy_set_header X-Forwarded-Proto $scheme;\n"
            "            proxy_connect_timeout 600s;\n            proxy_send_timeout 600s;\n"
            "            proxy_read_timeout 600s;\n            proxy_buffering off;\n"
            "        }\n    }\n}\n")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Generate docker-compose.yml for a vLLM multi-instance deployment on ROCm")
    ap.add_argument("--system-info", action="store_true", help="print the GPU section of the system-information step and exit")
    ap.add_argument("--num-instances", type=int, help="Number of vLLM instances")
    ap.add_argument("--tensor-parallel-size", type=int, help="Tensor parallel size")
    ap.add_argument("--pipeline-parallel-size", type=int, default=1, help="Pipeline parallel size (default: 1)")
    ap.add_argument("--container-name", help="Base container name")
    ap.add_argument("--model-path", help="Path to model")
    ap.add_argument("--model-name", help="Model name")
    ap.add_argument("--hf-directory", help="HuggingFace cache directory")
    ap.add_argument("--hf-token", default="", help="HuggingFace token")
    ap.add_argument("--extra-args", default="", help='Extra vLLM arguments (e.g. "--enable-expert-parallel")')
    ap.add_argument("--nginx-conf", default=None, help="Path to nginx config file (for multi-instance)")
    ap.add_argument("--output", "-o", help="Output docker-compose.yml file path")
    ap.add_argument("--nginx-conf-output", default=None, help="Output nginx.conf file path (for multi-instance)")
    ap.add_argument("--library-dir", default=None,
                    help="root of this repository on the host: mounted into every server so that its AWQ layers "
                         "run on libawq_mi355x.so")
    ap.add_argument("--image", default=ROCM_VLLM_IMAGE, help="server / client image")
    args = ap.parse_args(argv)
    if args.system_info:
        sys.stdout.write(system_info_gpu_section())
        return 0
    missing = [f for f in ("num_instances", "tensor_parallel_size", "container_name", "model_path", "model_name",
                           "hf_directory", "output") if getattr(args, f) is None]
    if missing:
        ap.error("the following arguments are required: " + ", ".join("--" + m.replace("_", "-") for m in missing))
    nginx_conf_path = None
    if args.num_instances > 1:
        if not args.nginx_conf_output:
            print("Error: --nginx-conf-output required for multi-instance setup", file=sys.stderr)
            return 1
        with open(args.nginx_conf_output, "w") as f:
            f.write(nginx_conf(args.num_instances))
        nginx_conf_path = os.path.abspath(args.nginx_conf_output)      # docker compose wants an absolute path
    stack = compose(args.num_instances, args.tensor_parallel_size, args.pipeline_parallel_size, args.container_name,
                    args.model_path, args.model_name, args.hf_directory, args.hf_token, nginx_conf_path,
                    args.extra_args, total_rocm_gpus(), args.library_dir, args.image)
    with open(args.output, "w") as f:
        f.write(to_yaml(stack))
    print(f"Generated docker-compose.yml: {args.output}")
    if nginx_conf_path:
        print(f"Generated nginx.conf: {nginx_conf_path}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
