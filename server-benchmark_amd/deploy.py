"""docker-compose description of the serving stack for an MI355X host.

ROCm counterpart of the deployment the harness generates (reference
utils/generate_compose.py:46-100 vLLM service, :103-118 nginx, :121-143 benchmark client,
:146-190 nginx.conf, :12-43 GPU count): the same services, ports, volumes, server command
and health check, with the GPU plumbing of a ROCm container (/dev/kfd + /dev/dri, group
`video`, `HIP_VISIBLE_DEVICES`) in place of the NVIDIA runtime reservation, and with this
library mounted into the server so that its AWQ layers run on it.  The stack is built as
plain data and serialised with yaml.safe_dump; nothing here talks to docker.
"""
from __future__ import annotations

import re
from typing import Optional

import yaml

ROCM_VLLM_IMAGE = "rocm/vllm:latest"
HEALTHCHECK = ("curl -f http://localhost:8000/health && "
               "curl -f http://localhost:8000/v1/models | grep -q 'object.*list'")


def count_rocm_gpus(rocminfo_text: str) -> int:
    """GPU agents in `rocminfo` output (agents whose Device Type is GPU)."""
    return len(re.findall(r"^\s*Device Type:\s+GPU\s*$", rocminfo_text, flags=re.M))


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
        # the package (with libawq_mi355x.so inside) next to the server's Python path; the
        # installed wheel's vllm.general_plugins entry point does the rebinding
        volumes.append(f"{library_dir}:/opt/awq_mi355x:ro")
        env.append("PYTHONPATH=/opt/awq_mi355x")
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
            library_dir: Optional[str] = None) -> dict:
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
                                             model_name, hf_directory, hf_token, extra_args, library_dir)
    if num_instances > 1 and nginx_conf_path:
        services["nginx"] = nginx_service(num_instances, nginx_conf_path)
    services["benchmark"] = benchmark_service(hf_directory, hf_token)
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
