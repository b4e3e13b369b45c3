"""Operator surface of the AWQ W4A16 path, keeping vLLM's names and argument order:

    awq_dequantize(qweight, scales, zeros, split_k_iters, thx, thy) -> fp16 [K, N]
    awq_gemm(input, qweight, scales, qzeros, split_k_iters)          -> fp16 [M, N]

plus the fused-MoE pieces (topk_softmax, moe_align_block_size, moe_awq_gemm, silu_and_mul,
moe_sum).  Each function checks dtype / device / contiguity / shape relations, then calls
the C ABI with raw device pointers on torch's current stream.  Tensors are torch tensors on a
ROCm device; torch is used for memory and streams only.
"""
from __future__ import annotations

import warnings

import torch

from . import _lib

MOE_TILE_M = 16
_WS_COUNTER_BYTES = 65536
_workspaces: dict = {}
_retired: list = []      # outgrown workspaces, kept because captured graphs may still point at them
_warned_split_k_iters = False
_gemm_ws_bytes: dict = {}  # (M, K, N, split) -> awqmi_gemm_workspace_bytes, asked once per shape
DEV_VARIANT_NO_DENSE = 1 << 25   # development variant bits of awq_gemm (include/awq_mi355x_dev.h)
DEV_VARIANT_DENSE = 1 << 26


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device) -> int:
    """Handle of torch's current stream on the device (the raw getter skips building a Stream
    object: these wrappers run once per layer call, so a microsecond counts at M = 1)."""
    if _raw_stream is not None:
        idx = device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream


def _need(t: torch.Tensor, name: str, dtype, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")


def _need_qweight(t: torch.Tensor) -> int:
    """qweight of a dense layer: int32 [K, N / 8] on the GPU, contiguous or with padded rows (unit
    stride along a row, a whole number of 16-byte groups from one row to the next: what
    pad_qweight_rows makes).  Returns the row pitch in words."""
    if not isinstance(t, torch.Tensor):
        raise TypeError("qweight must be a torch.Tensor")
    if t.dtype != torch.int32:
        raise ValueError(f"qweight must be {torch.int32}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"qweight must live on the GPU (got {t.device}); there is no CPU path")
    if t.dim() != 2:
        raise ValueError(f"qweight must have 2 dims, got shape {tuple(t.shape)}")
    if t.is_contiguous():
        return t.shape[1]
    if t.stride(1) != 1 or t.stride(0) < t.shape[1] or t.stride(0) % 4 != 0:
        raise ValueError("qweight must be contiguous, or row-padded (unit stride inside a row, a row pitch "
                         "that is a multiple of 4 words)")
    return t.stride(0)


ROW_PAD_WORDS = 32      # one 128-byte line


def pad_qweight_rows(qweight: torch.Tensor) -> torch.Tensor:
    """The same [K, N / 8] qweight as a view of a buffer whose rows are one 128-byte line further
    apart, when the packed row is a multiple of four lines (512 bytes) and at least 32 lines long;
    any other qweight is returned as it is.  Every wave of the skinny kernel reads one line per
    row: with rows a multiple of 1 KiB apart all its requests share address bits 7 - 9 and the
    launch streams 12 - 20 % slower than with any other row pitch (8192 x N layers, N from 49152 to
    65536); a multiple of 512 bytes costs 5 - 10 % (228- and 116-line rows).  Rows of fewer than 32
    lines (N < 8192) measured the same either way."""
    K, NW = qweight.shape
    if NW % 128 != 0 or NW < 1024 or not qweight.is_contiguous():
        return qweight
    buf = torch.empty((K, NW + ROW_PAD_WORDS), dtype=qweight.dtype, device=qweight.device)
    buf[:, NW:].zero_()
    view = buf[:, :NW]
    view.copy_(qweight)
    return view


def _awq_shapes(qweight, scales, qzeros, lead=0):
    K, NW = qweight.shape[lead], qweight.shape[lead + 1]
    N = NW * 8
    groups = scales.shape[lead]
    if groups <= 0 or K % groups != 0:
        raise ValueError(f"scales rows {groups} must divide K={K}")
    if tuple(scales.shape[lead:]) != (groups, N):
        raise ValueError(f"scales shape {tuple(scales.shape)} != [.., {groups}, {N}]")
    if tuple(qzeros.shape[lead:]) != (groups, NW):
        raise ValueError(f"qzeros shape {tuple(qzeros.shape)} != [.., {groups}, {NW}]")
    if lead and not (qweight.shape[0] == scales.shape[0] == qzeros.shape[0]):
        raise ValueError("expert dimension differs between qweight / scales / qzeros")
    return K, N, K // groups


def get_workspace(device, nbytes: int, stream_ptr: int | None = None) -> torch.Tensor:
    """Per (device, stream) zero-initialised workspace; the kernels leave the counter
    prefix zeroed, so it is reused call after call."""
    dev = device if isinstance(device, torch.device) else torch.device(device)
    if stream_ptr is None:
        stream_ptr = _stream_ptr(dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), stream_ptr)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if not _workspaces:
            # first GPU use in this process: the library's one-time set-up, so that no later
            # call (possibly inside a stream capture) has to do it
            _lib.check(_lib.load().awqmi_init(), "awqmi_init")
        if ws is not None:
            # a HIP graph captured earlier on this stream holds the old buffer's address: keep
            # it alive, and grow geometrically so that few buffers are ever retired
            _retired.append(ws)
            nbytes = max(nbytes, 2 * ws.numel())
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def awq_dequantize(qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                   split_k_iters: int = 0, thx: int = 0, thy: int = 0) -> torch.Tensor:
    """fp16 [K, N] = fp16((w - z) * s).  split_k_iters / thx / thy are accepted for
    signature compatibility and ignored."""
    ldw = _need_qweight(qweight)
    _need(scales, "scales", torch.float16, 2)
    _need(zeros, "zeros", torch.int32, 2)
    K, N, G = _awq_shapes(qweight, scales, zeros)
    out = torch.empty((K, N), dtype=torch.float16, device=qweight.device)
    lib = _lib.load()
    st = lib.awqmi_dequantize_ld_f16(qweight.data_ptr(), ldw, scales.data_ptr(), zeros.data_ptr(),
                                     out.data_ptr(), K, N, G, _stream_ptr(qweight.device))
    _lib.check(st, "awq_dequantize")
    return out


def awq_gemm(input: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
             qzeros: torch.Tensor, split_k_iters: int = 0, *, force_split_k: int | None = None,
             out: torch.Tensor | None = None, _dev_variant: int | None = None) -> torch.Tensor:
    """fp16 [M, N] = input[M, K] @ dequant(qweight, scales, qzeros).

    split_k_iters is accepted in vLLM's position and ignored, like thx / thy of awq_dequantize:
    vLLM's AWQLinearMethod.apply always passes its pack factor (8) there, a tuning value of its
    own kernel, and this library picks the split that fills the chip in one round of
    workgroups from the shape.  force_split_k (1 .. 64) forces a split-K factor for the skinny
    kernel; tests and sweeps use it.  _dev_variant routes the call through the library's
    development entry point (single launch rules switched off or forced)."""
    global _warned_split_k_iters
    if split_k_iters not in (0, 8) and not _warned_split_k_iters:
        _warned_split_k_iters = True
        warnings.warn(f"awq_gemm: split_k_iters={split_k_iters} is ignored (the library picks the split from the "
                      "shape); pass force_split_k= to force a factor", stacklevel=2)
    _need(input, "input", torch.float16, 2)
    ldw = _need_qweight(qweight)
    _need(scales, "scales", torch.float16, 2)
    _need(qzeros, "qzeros", torch.int32, 2)
    K, N, G = _awq_shapes(qweight, scales, qzeros)
    M = input.shape[0]
    if input.shape[1] != K:
        raise ValueError(f"input has K={input.shape[1]}, qweight has K={K}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=input.device)
    else:
        _need(out, "out", torch.float16, 2)
        if tuple(out.shape) != (M, N):
            raise ValueError("out has the wrong shape")
    if M == 0:
        return out
    lib = _lib.load()
    split = 0 if force_split_k is None else max(0, min(int(force_split_k), 64))
    shape_key = (M, K, N, split)
    nbytes = _gemm_ws_bytes.get(shape_key)
    if nbytes is None:
        nbytes = _gemm_ws_bytes[shape_key] = lib.awqmi_gemm_workspace_bytes(M, K, N, split)
    if _dev_variant is not None and _dev_variant >= 0 and (_dev_variant & DEV_VARIANT_DENSE):
        # the dequantise-once form forced below the row count at which the workspace query counts on it
        nbytes = max(nbytes, lib.awqmi_dev_gemm_dense_workspace_bytes(M, K, N))
    stream = _stream_ptr(input.device)
    ws = get_workspace(input.device, nbytes, stream)
    args = (input.data_ptr(), qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(),
            ws.data_ptr(), ws.numel(), M, K, N, G, split, stream)
    if ldw != N // 8:
        if _dev_variant is not None:
            raise ValueError("the development entry point takes a contiguous qweight")
        st = lib.awqmi_gemm_ld_f16(args[0], args[1], ldw, *args[2:])
    elif _dev_variant is None:
        st = lib.awqmi_gemm_f16(*args)
    else:
        st = lib.awqmi_dev_gemm_f16(*args, int(_dev_variant))
    _lib.check(st, "awq_gemm")
    return out


_noalloc_last_stream: dict = {}   # device index -> stream of the last awq_gemm_noalloc call


def awq_gemm_noalloc(input: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                     out: torch.Tensor, force_split_k: int | None = None) -> torch.Tensor:
    """awq_gemm into a caller-provided `out` through the library's allocation-free entry point:
    split-K counters and partial tiles live in a static device array inside the library, so
    neither this wrapper nor the library allocates.  qweight may be contiguous or row-padded (as
    AWQLinearMethod holds it after loading).  All such calls on one GPU share that array and must
    not overlap in time: when a call arrives on another stream than the previous one on that GPU,
    the wrapper first waits on the host for the previous stream (and refuses to do so inside a
    stream capture, where it cannot wait: callers on several streams use awq_gemm, whose workspace
    is per stream).  Raises ValueError when the call's split-K tiles do not fit."""
    _need(input, "input", torch.float16, 2)
    ldw = _need_qweight(qweight)
    _need(scales, "scales", torch.float16, 2)
    _need(qzeros, "qzeros", torch.int32, 2)
    _need(out, "out", torch.float16, 2)
    K, N, G = _awq_shapes(qweight, scales, qzeros)
    M = input.shape[0]
    if input.shape[1] != K or tuple(out.shape) != (M, N):
        raise ValueError(f"input {tuple(input.shape)} / out {tuple(out.shape)} do not fit K={K}, N={N}")
    if M == 0:
        return out
    split = 0 if force_split_k is None else max(0, min(int(force_split_k), 64))
    dev = input.device.index if input.device.index is not None else torch.cuda.current_device()
    stream = _stream_ptr(input.device)
    last = _noalloc_last_stream.get(dev)
    if last is not None and last != stream:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("awq_gemm_noalloc: the previous call on this GPU ran on another stream and this one is "
                               "being captured; the calls share one static scratch array and must be serialised "
                               "(use awq_gemm, whose workspace is per stream)")
        torch.cuda.ExternalStream(last, device=input.device).synchronize()
    _noalloc_last_stream[dev] = stream
    st = _lib.load().awqmi_gemm_f16_noalloc(input.data_ptr(), qweight.data_ptr(), ldw, scales.data_ptr(),
                                            qzeros.data_ptr(), out.data_ptr(), M, K, N, G, split, stream)
    _lib.check(st, "awq_gemm_noalloc")
    return out


def reset_workspace(device=None) -> None:
    """Zeroes the arrival counters of this (device, current stream)'s workspace.  Only needed
    after something cut a call short (a failed or aborted launch): calls that run to completion
    leave the counters at zero themselves."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    stream = _stream_ptr(dev)
    ws = get_workspace(dev, 1, stream)
    _lib.check(_lib.load().awqmi_workspace_reset(ws.data_ptr(), ws.numel(), stream), "reset_workspace")


# --------------------------------------------------------------------------- fused MoE

def topk_softmax(gating_output: torch.Tensor, topk: int, renormalize: bool = True):
    """softmax over experts then top-k.  Returns (topk_weights fp32 [T, k], topk_ids int32)."""
    _need(gating_output, "gating_output", torch.float32, 2)
    T, E = gating_output.shape
    ids = torch.empty((T, topk), dtype=torch.int32, device=gating_output.device)
    wts = torch.empty((T, topk), dtype=torch.float32, device=gating_output.device)
    if T == 0:
        return wts, ids
    st = _lib.load().awqmi_moe_topk_softmax_f32(gating_output.data_ptr(), T, E, topk, int(renormalize),
                                                ids.data_ptr(), wts.data_ptr(),
                                                _stream_ptr(gating_output.device))
    _lib.check(st, "topk_softmax")
    return wts, ids


def topk_route(gating_output: torch.Tensor, topk: int, renormalize: bool = True, scoring_func: str = "softmax",
               e_score_correction_bias: torch.Tensor | None = None, routed_scaling_factor: float = 1.0):
    """Routing with the scoring variants vLLM's fused MoE knows: "softmax" (plain top-k of the
    softmax) or "sigmoid" (experts chosen by sigmoid(logit) + e_score_correction_bias, weighted
    by sigmoid(logit)); weights optionally renormalised, then scaled.  Returns (weights, ids)."""
    _need(gating_output, "gating_output", torch.float32, 2)
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError(f"scoring_func must be 'softmax' or 'sigmoid', got {scoring_func!r}")
    T, E = gating_output.shape
    bias_ptr = 0
    if e_score_correction_bias is not None:
        if scoring_func != "sigmoid":
            raise ValueError("e_score_correction_bias goes with sigmoid scoring")
        _need(e_score_correction_bias, "e_score_correction_bias", torch.float32, 1)
        if e_score_correction_bias.shape[0] != E:
            raise ValueError(f"e_score_correction_bias has {e_score_correction_bias.shape[0]} entries, expected {E}")
        bias_ptr = e_score_correction_bias.data_ptr()
    ids = torch.empty((T, topk), dtype=torch.int32, device=gating_output.device)
    wts = torch.empty((T, topk), dtype=torch.float32, device=gating_output.device)
    if T == 0:
        return wts, ids
    st = _lib.load().awqmi_moe_topk_f32(gating_output.data_ptr(), bias_ptr, T, E, topk,
                                        1 if scoring_func == "sigmoid" else 0, int(renormalize),
                                        float(routed_scaling_factor), ids.data_ptr(), wts.data_ptr(),
                                        _stream_ptr(gating_output.device))
    _lib.check(st, "topk_route")
    return wts, ids


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Returns (sorted_token_ids, expert_ids, num_tokens_post_padded): flat slot indices
    stably sorted by expert, each expert's run padded to a multiple of block_size with the
    sentinel topk_ids.numel()."""
    _need(topk_ids, "topk_ids", torch.int32)
    n = topk_ids.numel()
    lib = _lib.load()
    cap = lib.awqmi_moe_align_capacity(n, num_experts, block_size)
    dev = topk_ids.device
    sorted_ids = torch.empty((cap,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((cap // block_size,), dtype=torch.int32, device=dev)
    npp = torch.empty((1,), dtype=torch.int32, device=dev)
    st = lib.awqmi_moe_align(topk_ids.data_ptr(), n, num_experts, block_size, sorted_ids.data_ptr(),
                             expert_ids.data_ptr(), npp.data_ptr(), _stream_ptr(dev))
    _lib.check(st, "moe_align_block_size")
    return sorted_ids, expert_ids, npp


def moe_awq_gemm(a: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                 sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                 num_tokens_post_padded: torch.Tensor, n_slots: int, a_row_div: int,
                 topk_weights: torch.Tensor | None = None, split_k: int = 0,
                 out: torch.Tensor | None = None, block_size: int = MOE_TILE_M,
                 _dev_variant: int | None = None) -> torch.Tensor:
    """Expert-grouped AWQ GEMM over blocks of `block_size` sorted slots (16 or 32: the skinny
    kernel; 64, 128 or 256: the MFMA kernel in its expert-grouped form, for many rows per expert):
    out[s] = a[s // a_row_div] @ W[expert(s)] (* topk_weights[s]).  The ids must come from
    moe_align_block_size with the same block size."""
    _need(a, "a", torch.float16, 2)
    _need(qweight, "qweight", torch.int32, 3)
    _need(scales, "scales", torch.float16, 3)
    _need(qzeros, "qzeros", torch.int32, 3)
    _need(sorted_token_ids, "sorted_token_ids", torch.int32, 1)
    _need(expert_ids, "expert_ids", torch.int32, 1)
    _need(num_tokens_post_padded, "num_tokens_post_padded", torch.int32, 1)
    K, N, G = _awq_shapes(qweight, scales, qzeros, lead=1)
    E = qweight.shape[0]
    if a.shape[1] != K:
        raise ValueError(f"a has K={a.shape[1]}, qweight has K={K}")
    if a.shape[0] * a_row_div < n_slots:
        raise ValueError("a has too few rows for n_slots / a_row_div")
    lib = _lib.load()
    if block_size not in (16, 32, 64, 128, 256):
        raise ValueError("block_size must be 16, 32, 64, 128 or 256")
    cap = lib.awqmi_moe_align_capacity(n_slots, E, block_size)
    if sorted_token_ids.numel() < cap or expert_ids.numel() < cap // block_size:
        raise ValueError("sorted_token_ids / expert_ids smaller than the align capacity")
    tw = 0
    if topk_weights is not None:
        _need(topk_weights, "topk_weights", torch.float32)
        if topk_weights.numel() < n_slots:
            raise ValueError("topk_weights has fewer entries than n_slots")
        tw = topk_weights.data_ptr()
    if out is None:
        out = torch.empty((n_slots, N), dtype=torch.float16, device=a.device)
    split = max(0, min(int(split_k), 64))
    nbytes = lib.awqmi_moe_gemm_workspace_bytes(n_slots, E, K, N, split, block_size)
    stream = _stream_ptr(a.device)
    ws = get_workspace(a.device, nbytes, stream)
    args = (a.data_ptr(), qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(),
            sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), tw, n_slots,
            a_row_div, block_size, E, K, N, G, split, ws.data_ptr(), ws.numel(), stream)
    if _dev_variant is None:
        st = lib.awqmi_moe_gemm_f16(*args)
    else:
        st = lib.awqmi_dev_moe_gemm_f16(*args, int(_dev_variant))
    _lib.check(st, "moe_awq_gemm")
    return out


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """[rows, 2I] ([gate | up]) -> silu(gate) * up, fp16 [rows, I]."""
    _need(x, "x", torch.float16, 2)
    rows, two_i = x.shape
    out = torch.empty((rows, two_i // 2), dtype=torch.float16, device=x.device)
    st = _lib.load().awqmi_silu_and_mul_f16(x.data_ptr(), out.data_ptr(), rows, two_i // 2,
                                           _stream_ptr(x.device))
    _lib.check(st, "silu_and_mul")
    return out


def moe_sum(x: torch.Tensor, T: int, topk: int) -> torch.Tensor:
    """[T * topk, H] -> [T, H], fp32 sum over a token's slots."""
    _need(x, "x", torch.float16, 2)
    H = x.shape[1]
    out = torch.empty((T, H), dtype=torch.float16, device=x.device)
    st = _lib.load().awqmi_moe_sum_f16(x.data_ptr(), out.data_ptr(), T, topk, H, _stream_ptr(x.device))
    _lib.check(st, "moe_sum")
    return out


def fused_moe_awq(hidden_states: torch.Tensor, w13, w2, gating_output: torch.Tensor, topk: int,
                  renormalize: bool = True, block_size: int | None = None, scoring_func: str = "softmax",
                  e_score_correction_bias: torch.Tensor | None = None,
                  routed_scaling_factor: float = 1.0, _dev_variant: int | None = None) -> torch.Tensor:
    """One AWQ MoE block: route -> align -> grouped GEMM (w13) -> SiLU*up -> grouped GEMM (w2,
    scaled by the routing weight) -> sum over slots.  w13 / w2 are (qweight, scales, qzeros)
    with a leading expert dimension; w13 columns are [gate | up].  With block_size left at
    None the block runs as one library call (softmax routing, or sigmoid scoring with an
    optional score-correction bias; routing weights times routed_scaling_factor); a block size
    selects the step-by-step path over blocks of that size."""
    _need(hidden_states, "hidden_states", torch.float16, 2)
    T, H = hidden_states.shape
    E = w13[0].shape[0]
    if T == 0:
        return hidden_states.new_empty((0, H))
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError(f"scoring_func must be 'softmax' or 'sigmoid', got {scoring_func!r}")
    if block_size is None:
        # the whole block in one library call, intermediates in the workspace
        for i, (t, dt) in enumerate(zip(tuple(w13) + tuple(w2), (torch.int32, torch.float16, torch.int32) * 2)):
            _need(t, f"w13/w2[{i}]", dt, 3)
        K1, N1, G1 = _awq_shapes(*w13, lead=1)
        K2, N2, G2 = _awq_shapes(*w2, lead=1)
        inter = N1 // 2
        if K1 != H or N2 != H or K2 != inter or N1 != 2 * inter or G1 != G2 or w2[0].shape[0] != E:
            raise ValueError(f"w13 [{K1}, {N1}] / w2 [{K2}, {N2}] do not fit hidden {H}")
        lg = gating_output
        if lg.dtype != torch.float32 or not lg.is_contiguous():
            lg = lg.float().contiguous()
        _need(lg, "gating_output", torch.float32, 2)
        if tuple(lg.shape) != (T, E):
            raise ValueError(f"gating_output shape {tuple(lg.shape)} != ({T}, {E})")
        bias = 0
        if e_score_correction_bias is not None:
            if scoring_func != "sigmoid":
                raise ValueError("e_score_correction_bias belongs to sigmoid scoring")
            bias_t = e_score_correction_bias
            if bias_t.dtype != torch.float32 or not bias_t.is_contiguous():
                bias_t = bias_t.float().contiguous()
            _need(bias_t, "e_score_correction_bias", torch.float32, 1)
            if bias_t.numel() != E:
                raise ValueError(f"e_score_correction_bias has {bias_t.numel()} entries for {E} experts")
            bias = bias_t.data_ptr()
        lib = _lib.load()
        nbytes = lib.awqmi_fused_moe_workspace_bytes(T, H, inter, E, topk)
        stream = _stream_ptr(hidden_states.device)
        ws = get_workspace(hidden_states.device, nbytes, stream)
        out = torch.empty((T, H), dtype=torch.float16, device=hidden_states.device)
        args = (hidden_states.data_ptr(), lg.data_ptr(), bias, w13[0].data_ptr(), w13[1].data_ptr(),
                w13[2].data_ptr(), w2[0].data_ptr(), w2[1].data_ptr(), w2[2].data_ptr(), out.data_ptr(), T, H,
                inter, E, topk, G1, 1 if scoring_func == "sigmoid" else 0, int(renormalize),
                float(routed_scaling_factor), ws.data_ptr(), ws.numel(), stream)
        if _dev_variant is None:
            st = lib.awqmi_fused_moe_routed_f16(*args)
        else:
            st = lib.awqmi_dev_fused_moe_routed_f16(*args, int(_dev_variant))
        _lib.check(st, "fused_moe_awq")
        return out
    T = hidden_states.shape[0]
    E = w13[0].shape[0]
    topk_w, topk_ids = topk_route(gating_output.float().contiguous(), topk, renormalize, scoring_func,
                                  e_score_correction_bias, routed_scaling_factor)
    n = T * topk
    # 16-row blocks measured faster than 32-row blocks at every token count tried (the
    # two-row-block instantiation of the skinny kernel is issue-bound)
    bs = block_size if block_size is not None else MOE_TILE_M
    sorted_ids, expert_ids, npp = moe_align_block_size(topk_ids, bs, E)
    h13 = moe_awq_gemm(hidden_states, *w13, sorted_ids, expert_ids, npp, n, topk, block_size=bs,
                       _dev_variant=_dev_variant)
    act = silu_and_mul(h13)
    o = moe_awq_gemm(act, *w2, sorted_ids, expert_ids, npp, n, 1, topk_weights=topk_w, block_size=bs,
                     _dev_variant=_dev_variant)
    return moe_sum(o, T, topk)
