"""Host side of the FP8 fused-MoE path: thin torch wrappers over the C ABI.

Tensors live on a ROCm device ("cuda" in PyTorch-ROCm); torch is used for memory and the
current stream only.  Every wrapper validates what the C side cannot see (dtype, device,
contiguity), passes raw pointers and the current HIP stream, and raises RuntimeError on a
non-zero return, as the reference's ops raise through TORCH_CHECK
(torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:143,148,231).
"""
from __future__ import annotations

import torch

from ._lib import MoeHipError, check, lib

ROUTE_SOFTMAX, ROUTE_SIGMOID, ROUTE_SCORES, ROUTE_SOFTMAX_LOGIT_BIAS = 0, 1, 2, 3
_FP8 = torch.float8_e4m3fn


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def _dev(t: torch.Tensor, name: str, dtype=None):
    _need(isinstance(t, torch.Tensor), f"{name} must be a tensor")
    _need(t.is_cuda, f"{name} must be on the GPU")
    _need(t.is_contiguous(), f"{name} must be contiguous")
    if dtype is not None:
        _need(t.dtype in (dtype if isinstance(dtype, tuple) else (dtype,)), f"{name} must be {dtype}, got {t.dtype}")
    return t.data_ptr()


def _dtype_sel(t: torch.Tensor, name: str) -> int:
    _need(t.dtype in (torch.float32, torch.bfloat16), f"{name} must be float32 or bfloat16")
    return 0 if t.dtype == torch.float32 else 1


def tile_rows(T: int, K: int, E: int) -> int:
    return lib.moe_tile_rows(T, K, E)


# --------------------------------------------------------------------------- routing
def noaux_tc_topk(values, indices, scores, n_groups: int, topk_groups: int, top_k: int):
    """Group-limited top-k into caller-allocated `values` / `indices`; returns `values`
    (signature of the reference op, torch_tpu/csrc/ops/my_ops/NoauxTcTopk.cpp:9-67)."""
    _need(scores.dim() == 2, "scores must be 2D tensor")
    _need(values.dtype == scores.dtype, "values and scores must have the same dtype")
    _need(indices.dtype == torch.int32, "indices must be int32")
    T, E = scores.shape
    _need(tuple(values.shape) == (T, top_k), "values shape must be [batch_size, top_k]")
    _need(tuple(indices.shape) == (T, top_k), "indices shape must be [batch_size, top_k]")
    _need(n_groups > 0 and E % n_groups == 0, "total_size must be divisible by n_groups")
    _need(topk_groups <= n_groups, "topk_groups must be <= n_groups")
    _need(top_k > 0, "top_k must be positive")
    sel = _dtype_sel(scores, "scores")
    rc = lib.moe_noaux_tc_topk(_stream(), _dev(scores, "scores"), sel, T, E, n_groups, topk_groups, top_k,
                               _dev(values, "values"), _dev(indices, "indices"))
    check(rc, "noaux_tc_topk")
    return values


def moe_route(logits, k: int, mode: str = "softmax", bias=None, n_groups: int = 1, topk_groups: int = 1,
              renorm: bool = True, scale: float = 1.0, return_scores: bool = False):
    """Top-k routing from router logits -> (fp32 weights [T,k], int32 ids [T,k][, fp32 scores [T,E]]).
    mode: "softmax" | "sigmoid" | "scores" (the input already holds scores)."""
    modes = {"softmax": ROUTE_SOFTMAX, "sigmoid": ROUTE_SIGMOID, "scores": ROUTE_SCORES,
             "softmax_logit_bias": ROUTE_SOFTMAX_LOGIT_BIAS}     # softmax over logits + bias (the bias is part of the logits)
    _need(mode in modes, f"unknown routing mode {mode!r}")
    _need(logits.dim() == 2, "logits must be [T, E]")
    T, E = logits.shape
    sel = _dtype_sel(logits, "logits")
    weights = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    scores = torch.empty(T, E, dtype=torch.float32, device=logits.device) if return_scores else None
    bias_ptr = None
    if bias is not None:
        _need(bias.numel() == E, "bias must hold one value per expert")
        bias_ptr = _dev(bias, "bias", torch.float32)
    rc = lib.moe_route_topk(_stream(), _dev(logits, "logits"), sel, bias_ptr, T, E, k, modes[mode], n_groups,
                            topk_groups, int(renorm), float(scale), weights.data_ptr(), ids.data_ptr(),
                            scores.data_ptr() if scores is not None else None)
    check(rc, "moe_route")
    return (weights, ids, scores) if return_scores else (weights, ids)


# --------------------------------------------------------------------------- permutation
def moe_permute(ids, num_experts: int, return_workspace: bool = False):
    """Stable counting sort of the flattened ids -> (sorted_slot [T*K], expert_offsets [E+1],
    slot_to_row [T*K]), all int32."""
    _need(ids.dim() == 2, "ids must be [T, K]")
    T, K = ids.shape
    dev = ids.device
    sorted_slot = torch.empty(T * K, dtype=torch.int32, device=dev)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    slot_to_row = torch.empty(T * K, dtype=torch.int32, device=dev)
    nbytes = lib.moe_permute_workspace_bytes(T, K, num_experts)
    _need(nbytes > 0, "bad permutation shape")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.moe_permute(_stream(), _dev(ids, "ids", torch.int32), T, K, num_experts, sorted_slot.data_ptr(),
                         offsets.data_ptr(), slot_to_row.data_ptr(), ws.data_ptr(), nbytes)
    check(rc, "moe_permute")
    if return_workspace:
        return sorted_slot, offsets, slot_to_row, ws
    return sorted_slot, offsets, slot_to_row


# --------------------------------------------------------------------------- quantisation
def scale_pitch(n_groups: int) -> int:
    """Floats per row of an activation-scale tensor holding n_groups scales per row."""
    return lib.moe_scale_pitch(n_groups)


def _new_scales(rows: int, n_groups: int, device):
    """[rows, n_groups] fp32 view of a freshly allocated row-padded scale tensor."""
    return torch.empty(rows, scale_pitch(n_groups), dtype=torch.float32, device=device)[:, :n_groups]


def _scales(t: torch.Tensor, name: str):
    """Device address of a scale tensor in the row-padded layout the kernels read; a tensor in any
    other layout is copied into a padded one first (returned so that it stays alive)."""
    _need(isinstance(t, torch.Tensor) and t.is_cuda and t.dim() == 2, f"{name} must be a 2-d GPU tensor")
    _need(t.dtype == torch.float32, f"{name} must be float32")
    rows, n = t.shape
    pitch = scale_pitch(n)
    room = t.untyped_storage().nbytes() - t.storage_offset() * 4 >= rows * pitch * 4
    if not (t.stride(1) == 1 and (rows <= 1 or t.stride(0) == pitch) and t.data_ptr() % 64 == 0 and room):
        padded = _new_scales(rows, n, t.device)
        padded.copy_(t)
        t = padded
    return t.data_ptr(), t


def act_quant(x):
    """bf16 [R, C] -> (e4m3fn [R, C], fp32 scales [R, C/128]: a view of a row-padded tensor)."""
    _need(x.dim() == 2, "x must be [R, C]")
    R, C = x.shape
    q = torch.empty(R, C, dtype=_FP8, device=x.device)
    s = _new_scales(R, C // 128, x.device)
    rc = lib.moe_act_quant(_stream(), _dev(x, "x", torch.bfloat16), R, C, q.data_ptr(), s.data_ptr())
    check(rc, "act_quant")
    return q, s


# --------------------------------------------------------------------------- weight layout
def _repack(w, fn, what):
    _need(isinstance(w, torch.Tensor) and w.dim() >= 2, f"{what}: weights must be [..., N, K]")
    _need(w.dtype in (_FP8, torch.bfloat16, torch.uint8), f"{what}: weights must be float8_e4m3fn, bfloat16 or uint8")
    N, K = w.shape[-2:]
    row_bytes = K * w.element_size()
    _need(N % 16 == 0 and row_bytes % 128 == 0, f"{what}: N must be a multiple of 16 and a row a multiple of 128 bytes")
    out = torch.empty_like(w)
    rows = w.numel() // K if K else 0
    check(fn(_stream(), _dev(w, "w"), rows, row_bytes, out.data_ptr()), what)
    return out


def pack_weights(w):
    """Row-major weights [..., N, K] on the GPU (N a multiple of 16, a row a multiple of 128 bytes) -> a tensor of the
    same shape and dtype whose bytes are in the tile-blocked order every GEMM entry point reads (see
    include/moe_hip.h).  Done once, when weights are loaded."""
    return _repack(w, lib.moe_pack_weights, "pack_weights")


def unpack_weights(w):
    """The inverse of pack_weights: tile-blocked bytes -> row-major."""
    return _repack(w, lib.moe_unpack_weights, "unpack_weights")


def pack_layer(w13, w13_scale, w2, w2_scale):
    """(w13, w13_scale, w2, w2_scale) with row-major weights on the GPU -> the same with tile-blocked weights."""
    return pack_weights(w13), w13_scale, pack_weights(w2), w2_scale


# --------------------------------------------------------------------------- experts
def _shared_args(shared, H: int):
    """(four device pointers, intermediate size) of an optional shared expert
    (w13 [1,2Is,H], w13_scale, w2 [1,H,Is], w2_scale); all None and 0 without one."""
    if shared is None:
        return [None, None, None, None], 0
    s13, s13s, s2, s2s = shared
    I_sh = s13.shape[1] // 2
    _need(tuple(s13.shape) == (1, 2 * I_sh, H) and tuple(s2.shape) == (1, H, I_sh), "bad shared expert shapes")
    _need(tuple(s13s.shape) == (1, 2 * I_sh // 128, H // 128) and tuple(s2s.shape) == (1, H // 128, I_sh // 128),
          "bad shared expert scale shapes")
    return [_dev(s13, "shared w13", _FP8), _dev(s13s, "shared w13 scale", torch.float32),
            _dev(s2, "shared w2", _FP8), _dev(s2s, "shared w2 scale", torch.float32)], I_sh


def fused_experts_workspace_bytes(T, H, I, E, K, I_shared=0) -> int:
    return lib.moe_fused_experts_workspace_bytes(T, H, I, E, K, I_shared)


def fused_experts_fp8(x, w13, w13_scale, w2, w2_scale, ids, routing_weights=None, out=None, shared=None,
                      workspace=None):
    """The expert computation on packed weights.

    x [T,H] bf16; w13 [E,2I,H] e4m3fn + fp32 scales [E,2I/128,H/128]; w2 [E,H,I] e4m3fn + fp32
    scales [E,H/128,I/128], both weight tensors TILE-BLOCKED (pack_weights); ids [T,K] int32.
    out [T,K,H] bf16: un-weighted per-slot results.  out [T,H] bf16: weighted sum over the
    slots (routing_weights fp32 [T,K] required), plus the shared expert
    shared=(w13 [1,2Is,H], w13_scale, w2 [1,H,Is], w2_scale) if given.
    Default out is [T,H] when routing_weights is given, else [T,K,H]."""
    _need(x.dim() == 2 and w13.dim() == 3 and w2.dim() == 3 and ids.dim() == 2, "bad ranks")
    T, H = x.shape
    E, I2, H2 = w13.shape
    I = I2 // 2
    K = ids.shape[1]
    _need(H2 == H and tuple(w2.shape) == (E, H, I), "weight shapes do not match x")
    _need(ids.shape[0] == T, "ids must be [T, K]")
    _need(H % 128 == 0 and I % 128 == 0, "H and I must be multiples of 128")
    _need(tuple(w13_scale.shape) == (E, I2 // 128, H // 128), "w13_scale must be [E, 2I/128, H/128]")
    _need(tuple(w2_scale.shape) == (E, H // 128, I // 128), "w2_scale must be [E, H/128, I/128]")
    if out is None:
        shape = (T, H) if routing_weights is not None else (T, K, H)
        out = torch.empty(shape, dtype=torch.bfloat16, device=x.device)
    mode = 1 if out.dim() == 2 else 0
    _need(tuple(out.shape) == ((T, H) if mode else (T, K, H)), "out must be [T,H] or [T,K,H]")
    rw_ptr = None
    if routing_weights is not None:
        _need(tuple(routing_weights.shape) == (T, K), "routing_weights must be [T, K]")
        rw_ptr = _dev(routing_weights, "routing_weights", torch.float32)
    _need(mode == 0 or rw_ptr is not None, "routing_weights are required for a [T,H] output")
    sh, I_sh = _shared_args(shared, H)
    need = fused_experts_workspace_bytes(T, H, I, E, K, I_sh)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_fused_experts_fp8(
        _stream(), _dev(x, "x", torch.bfloat16), T, H,
        _dev(w13, "w13", _FP8), _dev(w13_scale, "w13_scale", torch.float32),
        _dev(w2, "w2", _FP8), _dev(w2_scale, "w2_scale", torch.float32), I, E,
        _dev(ids, "ids", torch.int32), rw_ptr, K,
        sh[0], sh[1], sh[2], sh[3], I_sh,
        _dev(out, "out", torch.bfloat16), mode,
        _dev(workspace, "workspace"), workspace.numel() * workspace.element_size())
    check(rc, "fused_experts_fp8")
    return out


def set_shared_overlap(enabled: bool) -> bool:
    """Batches of 512 tokens and more: `layer_fp8` runs the shared expert's first GEMM on a stream of the library's
    own beside the router product, routing and permutation (same results bit for bit).  Returns the previous setting."""
    return bool(lib.moe_set_shared_overlap(1 if enabled else 0))


def layer_eligible(T: int, E: int, K: int) -> bool:
    """Shapes the one-call entry point takes (layer_fp8): any batch, up to 1024 experts."""
    return T >= 0 and 1 <= K <= E <= 1024


def router_logits(x, router_weight, out=None, workspace=None):
    """logits [T,E] bf16 = x [T,H] bf16 . router_weight [E,H]^T bf16 (fp32 sums, rounded once), E <= 1024."""
    _need(x.dim() == 2 and router_weight.dim() == 2 and x.shape[1] == router_weight.shape[1], "x must be [T,H], router_weight [E,H]")
    T, H = x.shape
    E = router_weight.shape[0]
    _need(E <= 1024 and H % 128 == 0, "router_logits takes E <= 1024 and H a multiple of 128")
    if out is None:
        out = torch.empty(T, E, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (T, E), "out must be [T, E]")
    need = lib.moe_router_logits_workspace_bytes(T, H, E)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_router_logits(_stream(), _dev(x, "x", torch.bfloat16), T, H, _dev(router_weight, "router_weight", torch.bfloat16),
                               E, _dev(out, "out", torch.bfloat16), _dev(workspace, "workspace"),
                               workspace.numel() * workspace.element_size())
    check(rc, "router_logits")
    return out


def layer_workspace_bytes(T, H, I, E, K, I_shared=0) -> int:
    return lib.moe_layer_fp8_workspace_bytes(T, H, I, E, K, I_shared)


def layer_fp8(x, router_weight, w13, w13_scale, w2, w2_scale, top_k: int, mode: str = "softmax", bias=None,
                     n_groups: int = 1, topk_groups: int = 1, renorm: bool = True, scale: float = 1.0, shared=None,
                     out=None, workspace=None, return_routing: bool = False, static_scratch: bool = False):
    """Router and experts of one layer in one call (E <= 1024).

    x [T,H] bf16, router_weight [E,H] bf16, the expert weights as in fused_experts_fp8.  Returns out [T,H] bf16,
    or (out, logits bf16 [T,E], weights fp32 [T,k], ids int32 [T,k]) with return_routing.
    static_scratch: use the library's built-in scratch array instead of a workspace (moe_layer_fp8_static: no
    device allocation when `out` is given; small batches only, calls on one GPU must not overlap)."""
    modes = {"softmax": ROUTE_SOFTMAX, "sigmoid": ROUTE_SIGMOID, "softmax_logit_bias": ROUTE_SOFTMAX_LOGIT_BIAS}
    _need(mode in modes, f"unknown routing mode {mode!r}")
    _need(x.dim() == 2 and w13.dim() == 3 and w2.dim() == 3 and router_weight.dim() == 2, "bad ranks")
    T, H = x.shape
    E, I2, H2 = w13.shape
    I = I2 // 2
    _need(layer_eligible(T, E, top_k), "layer_fp8 takes E <= 1024 and top_k <= E")
    _need(H2 == H and tuple(w2.shape) == (E, H, I) and tuple(router_weight.shape) == (E, H), "weight shapes do not match x")
    _need(H % 128 == 0 and I % 128 == 0, "H and I must be multiples of 128")
    _need(tuple(w13_scale.shape) == (E, I2 // 128, H // 128), "w13_scale must be [E, 2I/128, H/128]")
    _need(tuple(w2_scale.shape) == (E, H // 128, I // 128), "w2_scale must be [E, H/128, I/128]")
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (T, H), "out must be [T, H]")
    bias_ptr = None
    if bias is not None:
        _need(bias.numel() == E, "bias must hold one value per expert")
        bias_ptr = _dev(bias, "bias", torch.float32)
    sh, I_sh = _shared_args(shared, H)
    if not static_scratch:
        need = layer_workspace_bytes(T, H, I, E, top_k, I_sh)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
        _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    logits = weights = ids = None
    if return_routing:
        logits = torch.empty(T, E, dtype=torch.bfloat16, device=x.device)
        weights = torch.empty(T, top_k, dtype=torch.float32, device=x.device)
        ids = torch.empty(T, top_k, dtype=torch.int32, device=x.device)
    args = [
        _stream(), _dev(x, "x", torch.bfloat16), T, H, _dev(router_weight, "router_weight", torch.bfloat16), bias_ptr,
        E, top_k, modes[mode], n_groups, topk_groups, int(renorm), float(scale),
        _dev(w13, "w13", _FP8), _dev(w13_scale, "w13_scale", torch.float32),
        _dev(w2, "w2", _FP8), _dev(w2_scale, "w2_scale", torch.float32), I,
        sh[0], sh[1], sh[2], sh[3], I_sh, _dev(out, "out", torch.bfloat16),
        logits.data_ptr() if return_routing else None, weights.data_ptr() if return_routing else None,
        ids.data_ptr() if return_routing else None]
    if static_scratch:
        with torch.cuda.device(x.device):        # the array's address is looked up for the current device
            rc = lib.moe_layer_fp8_static(*args)
    else:
        rc = lib.moe_layer_fp8(*args, _dev(workspace, "workspace"), workspace.numel() * workspace.element_size())
    check(rc, "layer_fp8")
    return (out, logits, weights, ids) if return_routing else out


def fused_experts_bf16_workspace_bytes(T, H, I, E, K) -> int:
    return lib.moe_fused_experts_bf16_workspace_bytes(T, H, I, E, K)


def mm_workspace_bytes(M, K, N) -> int:
    return lib.moe_mm_fp8_workspace_bytes(M, K, N)


def mlp_workspace_bytes(M, H, I) -> int:
    return lib.moe_mlp_fp8_workspace_bytes(M, H, I)


def router_logits_workspace_bytes(T, H, E) -> int:
    return lib.moe_router_logits_workspace_bytes(T, H, E)


def fused_experts_bf16(x, w13, w2, ids, routing_weights=None, out=None, workspace=None):
    """The expert computation on un-quantised weights: x [T,H] bf16, w13 [E,2I,H] bf16 (gate rows, then
    up rows), w2 [E,H,I] bf16, ids [T,K] int32.  out [T,K,H]: per-slot results; out [T,H]: weighted sum."""
    _need(x.dim() == 2 and w13.dim() == 3 and w2.dim() == 3 and ids.dim() == 2, "bad ranks")
    T, H = x.shape
    E, I2, _ = w13.shape
    I = I2 // 2
    K = ids.shape[1]
    _need(tuple(w13.shape) == (E, 2 * I, H) and tuple(w2.shape) == (E, H, I), "w13 must be [E,2I,H] and w2 [E,H,I]")
    _need(ids.shape[0] == T, "ids must be [T, K]")
    if out is None:
        out = torch.empty((T, K, H) if routing_weights is None else (T, H), dtype=torch.bfloat16, device=x.device)
    mode = 1 if out.dim() == 2 else 0
    _need(tuple(out.shape) == ((T, H) if mode else (T, K, H)), "out must be [T,H] or [T,K,H]")
    rw_ptr = None
    if routing_weights is not None:
        _need(tuple(routing_weights.shape) == (T, K), "routing_weights must be [T, K]")
        rw_ptr = _dev(routing_weights, "routing_weights", torch.float32)
    _need(mode == 0 or rw_ptr is not None, "routing_weights are required for a [T,H] output")
    need = lib.moe_fused_experts_bf16_workspace_bytes(T, H, I, E, K)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_fused_experts_bf16(_stream(), _dev(x, "x", torch.bfloat16), T, H, _dev(w13, "w13", torch.bfloat16),
                                    _dev(w2, "w2", torch.bfloat16), I, E, _dev(ids, "ids", torch.int32), rw_ptr, K,
                                    _dev(out, "out", torch.bfloat16), mode, _dev(workspace, "workspace"),
                                    workspace.numel() * workspace.element_size())
    check(rc, "fused_experts_bf16")
    return out


def fused_experts_w8a16(x, w13, w13_scale, w2, w2_scale, ids, routing_weights=None, out=None, workspace=None):
    """The expert computation in the reference's own arithmetic on the packed FP8 weights: bf16 activations, weights
    de-quantised in registers to bf16(float(code) * block scale), bf16 intermediate - no activation quantisation.
    Same tensors as fused_experts_fp8 (tile-blocked codes, fp32 block scales), workspace of fused_experts_bf16."""
    _need(x.dim() == 2 and w13.dim() == 3 and w2.dim() == 3 and ids.dim() == 2, "bad ranks")
    T, H = x.shape
    E, I2, _ = w13.shape
    I = I2 // 2
    K = ids.shape[1]
    _need(tuple(w13.shape) == (E, 2 * I, H) and tuple(w2.shape) == (E, H, I), "w13 must be [E,2I,H] and w2 [E,H,I]")
    _need(H % 128 == 0 and I % 128 == 0, "H and I must be multiples of 128")
    _need(tuple(w13_scale.shape) == (E, 2 * I // 128, H // 128) and tuple(w2_scale.shape) == (E, H // 128, I // 128),
          "bad scale shapes")
    _need(ids.shape[0] == T, "ids must be [T, K]")
    if out is None:
        out = torch.empty((T, K, H) if routing_weights is None else (T, H), dtype=torch.bfloat16, device=x.device)
    mode = 1 if out.dim() == 2 else 0
    _need(tuple(out.shape) == ((T, H) if mode else (T, K, H)), "out must be [T,H] or [T,K,H]")
    rw_ptr = None
    if routing_weights is not None:
        _need(tuple(routing_weights.shape) == (T, K), "routing_weights must be [T, K]")
        rw_ptr = _dev(routing_weights, "routing_weights", torch.float32)
    _need(mode == 0 or rw_ptr is not None, "routing_weights are required for a [T,H] output")
    need = lib.moe_fused_experts_bf16_workspace_bytes(T, H, I, E, K)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_fused_experts_w8a16(_stream(), _dev(x, "x", torch.bfloat16), T, H, _dev(w13, "w13", _FP8),
                                     _dev(w13_scale, "w13_scale", torch.float32), _dev(w2, "w2", _FP8),
                                     _dev(w2_scale, "w2_scale", torch.float32), I, E, _dev(ids, "ids", torch.int32),
                                     rw_ptr, K, _dev(out, "out", torch.bfloat16), mode, _dev(workspace, "workspace"),
                                     workspace.numel() * workspace.element_size())
    check(rc, "fused_experts_w8a16")
    return out


# --------------------------------------------------------------------------- dense layers
def mm_fp8(x, w, w_scale, out=None, workspace=None):
    """Dense block-scaled linear layer: x [M,K] bf16, w [N,K] e4m3fn, fp32 scales [ceil(N/128), K/128]
    -> out [M,N] bf16.  The activations are quantised per row and 128 columns first."""
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x must be [M,K] and w [N,K]")
    M, K = x.shape
    N = w.shape[0]
    _need(tuple(w_scale.shape) == ((N + 127) // 128, K // 128), "w_scale must be [ceil(N/128), K/128]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (M, N), "out must be [M,N]")
    need = lib.moe_mm_fp8_workspace_bytes(M, K, N)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_mm_fp8(_stream(), _dev(x, "x", torch.bfloat16), M, K, _dev(w, "w", _FP8),
                        _dev(w_scale, "w_scale", torch.float32), N, _dev(out, "out", torch.bfloat16),
                        _dev(workspace, "workspace"), workspace.numel() * workspace.element_size())
    check(rc, "mm_fp8")
    return out


def mm_bf16(x, w, out=None):
    """Dense linear layer on un-quantised operands: x [M,K] bf16, w [N,K] bf16 -> out [M,N] bf16."""
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x must be [M,K] and w [N,K]")
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (M, N), "out must be [M,N]")
    rc = lib.moe_mm_bf16(_stream(), _dev(x, "x", torch.bfloat16), M, K, _dev(w, "w", torch.bfloat16), N,
                         _dev(out, "out", torch.bfloat16))
    check(rc, "mm_bf16")
    return out


def mm_w8a16(x, w, w_scale, out=None):
    """Dense block-scaled linear layer in the reference's arithmetic: x [M,K] bf16 (not quantised), w [N,K] e4m3fn
    (tile-blocked) de-quantised in registers to bf16(float(code) * scale), fp32 scales [ceil(N/128), K/128]
    -> out [M,N] bf16."""
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x must be [M,K] and w [N,K]")
    M, K = x.shape
    N = w.shape[0]
    _need(K % 128 == 0, "K must be a multiple of 128")
    _need(tuple(w_scale.shape) == ((N + 127) // 128, K // 128), "w_scale must be [ceil(N/128), K/128]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (M, N), "out must be [M,N]")
    rc = lib.moe_mm_w8a16(_stream(), _dev(x, "x", torch.bfloat16), M, K, _dev(w, "w", _FP8),
                          _dev(w_scale, "w_scale", torch.float32), N, _dev(out, "out", torch.bfloat16))
    check(rc, "mm_w8a16")
    return out


def mlp_fp8(x, w13, w13_scale, w2, w2_scale, out=None, workspace=None):
    """Dense gated MLP: x [M,H] bf16, w13 [2I,H] (gate rows then up rows), w2 [H,I], fp32 128x128
    block scales -> out [M,H] bf16 = (silu(x Wg^T) * (x Wu^T)) Wd^T, FP8 matrix products."""
    _need(x.dim() == 2 and w13.dim() == 2 and w2.dim() == 2, "x, w13, w2 must be 2-d")
    M, H = x.shape
    I = w13.shape[0] // 2
    _need(tuple(w13.shape) == (2 * I, H) and tuple(w2.shape) == (H, I), "w13 must be [2I,H] and w2 [H,I]")
    _need(tuple(w13_scale.shape) == (2 * I // 128, H // 128) and tuple(w2_scale.shape) == (H // 128, I // 128),
          "bad scale shapes")
    if out is None:
        out = torch.empty(M, H, dtype=torch.bfloat16, device=x.device)
    _need(tuple(out.shape) == (M, H), "out must be [M,H]")
    need = lib.moe_mlp_fp8_workspace_bytes(M, H, I)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _need(workspace.numel() * workspace.element_size() >= need, "workspace too small")
    rc = lib.moe_mlp_fp8(_stream(), _dev(x, "x", torch.bfloat16), M, H, _dev(w13, "w13", _FP8),
                         _dev(w13_scale, "w13_scale", torch.float32), _dev(w2, "w2", _FP8),
                         _dev(w2_scale, "w2_scale", torch.float32), I, _dev(out, "out", torch.bfloat16),
                         _dev(workspace, "workspace"), workspace.numel() * workspace.element_size())
    check(rc, "mlp_fp8")
    return out


def gemm1_swiglu(xq, xs, w13, w13_scale, ids_shape, sorted_slot, offsets, permute_ws):
    """Stage: first grouped GEMM + SwiGLU + re-quantisation -> (hq [T*K, I] e4m3fn, hs [T*K, I/128])."""
    T, K = ids_shape
    E, I2, H = w13.shape
    I = I2 // 2
    hq = torch.empty(T * K, I, dtype=_FP8, device=xq.device)
    hs = _new_scales(T * K, I // 128, xq.device)
    xs_ptr, xs = _scales(xs, "xs")
    rc = lib.moe_gemm1_swiglu(_stream(), _dev(xq, "xq", _FP8), xs_ptr, T, H,
                              _dev(w13, "w13", _FP8), _dev(w13_scale, "w13_scale", torch.float32), I, E, K,
                              _dev(sorted_slot, "sorted_slot", torch.int32), _dev(offsets, "offsets", torch.int32),
                              _dev(permute_ws, "permute_ws"), hq.data_ptr(), hs.data_ptr())
    check(rc, "gemm1_swiglu")
    return hq, hs


def gemm2(hq, hs, w2, w2_scale, ids_shape, sorted_slot, offsets, permute_ws, y=None):
    """Stage: second grouped GEMM -> y [T, K, H] bf16 (slot order)."""
    T, K = ids_shape
    E, H, I = w2.shape
    if y is None:
        y = torch.empty(T, K, H, dtype=torch.bfloat16, device=hq.device)
    hs_ptr, hs = _scales(hs, "hs")
    rc = lib.moe_gemm2(_stream(), _dev(hq, "hq", _FP8), hs_ptr, T, H,
                       _dev(w2, "w2", _FP8), _dev(w2_scale, "w2_scale", torch.float32), I, E, K,
                       _dev(sorted_slot, "sorted_slot", torch.int32), _dev(offsets, "offsets", torch.int32),
                       _dev(permute_ws, "permute_ws"), _dev(y, "y", torch.bfloat16))
    check(rc, "gemm2")
    return y


def weighted_reduce(y, routing_weights, shared_y=None, out=None):
    T, K, H = y.shape
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=y.device)
    rc = lib.moe_weighted_reduce(_stream(), _dev(y, "y", torch.bfloat16),
                                 _dev(routing_weights, "routing_weights", torch.float32),
                                 _dev(shared_y, "shared_y", torch.bfloat16) if shared_y is not None else None,
                                 T, K, H, _dev(out, "out", torch.bfloat16))
    check(rc, "weighted_reduce")
    return out


__all__ = ["MoeHipError", "noaux_tc_topk", "moe_route", "moe_permute", "act_quant", "fused_experts_fp8",
           "pack_weights", "unpack_weights", "pack_layer",
           "fused_experts_workspace_bytes", "gemm1_swiglu", "gemm2", "weighted_reduce", "tile_rows"]
