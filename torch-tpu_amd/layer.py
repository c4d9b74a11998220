"""Weight packing and a module-shaped wrapper around the fused-MoE path.

The reference passes three separate weight tensors per call: gate [E,I,H], up [E,I,H] and a
PRE-TRANSPOSED down [E,I,H], with bf16 block scales of matching orientation
(python/regression/test_llm/test_moe.py:285-288).  The kernels here want the reduction
dimension contiguous for both GEMMs and the weight bytes in matrix-instruction operand order, so
weights are packed once, at load time: W13 = gate rows followed by up rows [E,2I,H], W2 = down in
its checkpoint orientation [E,H,I], scales widened to fp32, then the bytes of W13 and W2 tile-blocked
(ops.pack_weights).
"""
from __future__ import annotations

import torch

from . import ops


def _pad_to(t, rows: int, cols: int):
    """Zero-pads the last two dimensions of t up to [rows, cols] (code 0 is +0.0 in e4m3fn as in every float type)."""
    r, c = t.shape[-2:]
    if r == rows and c == cols:
        return t
    if t.dtype == torch.float8_e4m3fn:
        return torch.nn.functional.pad(t.view(torch.uint8), (0, cols - c, 0, rows - r)).view(torch.float8_e4m3fn)
    return torch.nn.functional.pad(t, (0, cols - c, 0, rows - r))


def stack_expert_weights(gate, up, down_t, gate_scale, up_scale, down_t_scale):
    """Reference-layout fp8 weights -> (w13, w13_scale, w2, w2_scale), ROW-MAJOR: gate rows followed by up rows,
    down back in its checkpoint orientation, scales widened to fp32.  Pure data movement (concatenate / transpose /
    widen) on whatever device the tensors live; values are untouched.

    H or I that 128 does not divide (the reference de-quantises ceil(n/128) blocks, the last one partial:
    torch_tpu/csrc/ops/my_ops/fusedMoE.pl:11-34): gate, up and down are padded with zero codes to the next multiple
    of 128 in both dimensions - the scale tensors already hold ceil(n/128) blocks - so that every block is whole;
    zero weights add nothing to any sum, and a caller pads the activations' columns the same way."""
    I, H = gate.shape[-2:]
    Ip, Hp = -(-I // 128) * 128, -(-H // 128) * 128
    w13 = torch.cat([_pad_to(gate, Ip, Hp), _pad_to(up, Ip, Hp)], dim=1).contiguous()
    w13_scale = torch.cat([gate_scale, up_scale], dim=1).to(torch.float32).contiguous()
    w2 = _pad_to(down_t, Ip, Hp).transpose(1, 2).contiguous()
    w2_scale = down_t_scale.transpose(1, 2).to(torch.float32).contiguous()
    return w13, w13_scale, w2, w2_scale


def pack_expert_weights(gate, up, down_t, gate_scale, up_scale, down_t_scale):
    """Reference-layout fp8 weights on the GPU -> (w13, w13_scale, w2, w2_scale) in kernel layout: stacked as
    stack_expert_weights does, then the weight bytes tile-blocked (ops.pack_weights).  Values are untouched."""
    return ops.pack_layer(*stack_expert_weights(gate, up, down_t, gate_scale, up_scale, down_t_scale))


def quant_weight_block128(w: torch.Tensor):
    """bf16/fp32 weights [..., N, K] (N, K multiples of 128) -> (e4m3fn codes, fp32 scale per
    128x128 block), scale = max(amax, 1e-10) / 448, codes = clamp(w / scale, +-448) rounded to
    nearest even.  Runs wherever `w` lives; meant for converting a checkpoint once."""
    N, K = w.shape[-2:]
    if N % 128 or K % 128:
        raise RuntimeError("weight dimensions must be multiples of 128")
    lead = w.shape[:-2]
    blk = w.to(torch.float32).reshape(*lead, N // 128, 128, K // 128, 128)
    scale = blk.abs().amax(dim=(-3, -1)).clamp_min(1e-10) / 448.0
    q = (blk / scale[..., :, None, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.reshape(*lead, N, K), scale


def synthetic_weights(n_experts: int, n: int, k: int, device, seed: int, std: float = 0.02, tile_block: bool = True):
    """Random weights [n_experts, n, k] ~ N(0, std) in bf16, quantised to e4m3fn with fp32 128x128 block scales on
    `device`, in slices of experts (the fp32 intermediates of a whole layer are large) -> (codes, scales); the codes
    tile-blocked unless tile_block=False.  For benchmarks and tests: there are no checkpoints offline."""
    g = torch.Generator(device=device).manual_seed(seed)
    q = torch.empty(n_experts, n, k, dtype=torch.float8_e4m3fn, device=device)
    s = torch.empty(n_experts, n // 128, k // 128, dtype=torch.float32, device=device)
    step = max(1, (1 << 27) // (n * k))
    for e0 in range(0, n_experts, step):
        e1 = min(n_experts, e0 + step)
        w = (torch.randn(e1 - e0, n, k, generator=g, device=device) * std).to(torch.bfloat16)
        q[e0:e1], s[e0:e1] = quant_weight_block128(w)
    return (ops.pack_weights(q) if tile_block else q), s


def convert_hf_moe_layer(state: dict, prefix: str, num_experts: int, device=None, tile_block: bool = True):
    """Checkpoint tensors of one DeepSeek-V3-style FP8 MoE layer -> the packed layout of the kernels.
    tile_block=False stops before the last step (re-ordering the weight bytes on the GPU, ops.pack_weights) and
    returns the stacked row-major tensors, on any device.

    Reads `{prefix}experts.{e}.{gate,up,down}_proj.weight` (e4m3fn `[out, in]`) and the matching
    `.weight_scale_inv` (fp32 `[ceil(out/128), ceil(in/128)]`, the value a block is MULTIPLIED by),
    `{prefix}gate.weight` (router, `[E, H]`), optionally `{prefix}gate.e_score_correction_bias` and
    `{prefix}shared_experts.*`.  Returns a dict with router_weight, bias, w13, w13_scale, w2, w2_scale
    and shared (a 4-tuple or None).  Pure data movement: codes and scales are not re-quantised.
    The reference hands the same tensors to its op as separate gate / up / transposed-down arguments
    (python/regression/test_llm/test_moe.py:285-288); torch_tpu_amd.pack_expert_weights packs that form."""
    def get(name):
        t = state[prefix + name]
        return t.to(device) if device is not None else t

    if tile_block and device is None and not state[prefix + "gate.weight"].is_cuda:
        raise RuntimeError("convert_hf_moe_layer: tile-blocking the weight bytes runs on the GPU - pass device='cuda' "
                           "(or tile_block=False for the stacked row-major tensors on the host)")

    def stack(proj, suffix):
        return torch.stack([get(f"experts.{e}.{proj}.{suffix}") for e in range(num_experts)])

    # I or H that 128 does not divide: zero codes up to whole 128-blocks in both dimensions, as stack_expert_weights
    # does for the reference's argument form (the scale tensors already hold ceil(n/128) blocks)
    def whole(t):
        n, k = t.shape[-2:]
        return _pad_to(t, -(-n // 128) * 128, -(-k // 128) * 128)

    gate, up, down = stack("gate_proj", "weight"), stack("up_proj", "weight"), stack("down_proj", "weight")
    for t in (gate, up, down):
        if t.dtype != torch.float8_e4m3fn:
            raise RuntimeError("expert weights must be float8_e4m3fn (convert bf16 checkpoints with quant_weight_block128)")
    w13 = torch.cat([whole(gate), whole(up)], dim=1).contiguous()
    w13_scale = torch.cat([stack("gate_proj", "weight_scale_inv"), stack("up_proj", "weight_scale_inv")],
                          dim=1).to(torch.float32).contiguous()
    w2 = whole(down).contiguous()
    w2_scale = stack("down_proj", "weight_scale_inv").to(torch.float32).contiguous()
    shared = None
    if prefix + "shared_experts.gate_proj.weight" in state:
        sg, su, sd = (whole(get(f"shared_experts.{p}.weight")) for p in ("gate_proj", "up_proj", "down_proj"))
        sgs, sus, sds = (get(f"shared_experts.{p}.weight_scale_inv") for p in ("gate_proj", "up_proj", "down_proj"))
        shared = (torch.cat([sg, su], 0)[None].contiguous(), torch.cat([sgs, sus], 0)[None].to(torch.float32).contiguous(),
                  sd[None].contiguous(), sds[None].to(torch.float32).contiguous())
    bias = state.get(prefix + "gate.e_score_correction_bias")
    if bias is not None:
        bias = (bias.to(device) if device is not None else bias).to(torch.float32).contiguous()
    if tile_block:
        w13, w2 = ops.pack_weights(w13), ops.pack_weights(w2)
        if shared is not None:
            shared = ops.pack_layer(*shared)
    return dict(router_weight=get("gate.weight").to(torch.bfloat16).contiguous(), bias=bias, w13=w13, w13_scale=w13_scale,
                w2=w2, w2_scale=w2_scale, shared=shared)


class FusedMoE:
    """Router + routed experts (+ shared expert) of one MoE layer, inference only.

    Mirrors how the reference's tests wrap the op in a module holding the weights
    (python/regression/test_llm/test_moe.py:143-160), with the routing recipe of its callers
    (python/regression/test_llm/test_torch_ops.py:441-456) in front.
    """

    def __init__(self, router_weight, w13, w13_scale, w2, w2_scale, top_k, mode="softmax", bias=None,
                 n_groups=1, topk_groups=1, renorm=True, scale=1.0, shared=None):
        # w13 / w2 (and the shared expert's) are tile-blocked: ops.pack_weights / pack_expert_weights / convert_hf_moe_layer
        # [E, H]; the logits are a bf16 product (fp32 sums, rounded once) as in the reference's recipe
        # (python/regression/test_llm/test_torch_ops.py:440), so a router weight kept in fp32 is rounded once, here
        self.router_weight = router_weight if router_weight.dtype == torch.bfloat16 else router_weight.to(torch.bfloat16)
        self.w13, self.w13_scale, self.w2, self.w2_scale = w13, w13_scale, w2, w2_scale
        self.top_k, self.mode, self.bias = top_k, mode, bias
        self.n_groups, self.topk_groups, self.renorm, self.scale = n_groups, topk_groups, renorm, scale
        self.shared = shared
        self._ws = None

    def _workspace(self, T, decode=False):
        E, I2, H = self.w13.shape
        I_sh = self.shared[0].shape[1] // 2 if self.shared is not None else 0
        size = ops.layer_workspace_bytes if decode else ops.fused_experts_workspace_bytes
        need = size(T, H, I2 // 2, E, self.top_k, I_sh)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.w13.device)
        return self._ws

    def route(self, x):
        """The staged road: the router product and the selection as two calls (the kernels the one-call entry point
        runs for batches beyond the decode size) -> (weights fp32 [T,K], ids int32 [T,K])."""
        logits = ops.router_logits(x, self.router_weight)
        return ops.moe_route(logits, self.top_k, self.layer_mode(), self.bias, self.n_groups, self.topk_groups,
                             self.renorm, self.scale)

    def experts(self, x, weights, ids, out=None):
        return ops.fused_experts_fp8(x, self.w13, self.w13_scale, self.w2, self.w2_scale, ids, weights, out=out,
                                     shared=self.shared, workspace=self._workspace(x.shape[0]))

    def _one_call(self, T):
        return ops.layer_eligible(T, self.w13.shape[0], self.top_k)

    def layer_mode(self):
        """The routing mode handed to the one-call entry point: a softmax router's bias is part of the logits."""
        return "softmax_logit_bias" if self.mode == "softmax" and self.bias is not None else self.mode

    def __call__(self, x, out=None):
        T = x.shape[0]
        if self._one_call(T):      # router and experts behind one entry point
            return ops.layer_fp8(x, self.router_weight, self.w13, self.w13_scale, self.w2, self.w2_scale,
                                        self.top_k, self.layer_mode(), self.bias, self.n_groups, self.topk_groups, self.renorm,
                                        self.scale, shared=self.shared, out=out, workspace=self._workspace(T, True))
        weights, ids = self.route(x)
        return self.experts(x, weights, ids, out)


class FusedMoEModule(torch.nn.Module):
    """FusedMoE as a torch.nn.Module, the shape the reference's tests give their wrapper around the op
    (python/regression/test_llm/test_moe.py:143-160): the packed weights are buffers (so `.to(device)`, `state_dict()` and
    `load_state_dict()` see them), `forward(x)` = router -> experts (+ shared expert) -> [T, H] bf16.  Inference only."""

    def __init__(self, router_weight, w13, w13_scale, w2, w2_scale, top_k, mode="softmax", bias=None, n_groups=1,
                 topk_groups=1, renorm=True, scale=1.0, shared=None):
        super().__init__()
        self.register_buffer("router_weight", router_weight if router_weight.dtype == torch.bfloat16
                             else router_weight.to(torch.bfloat16))
        for name, t in (("w13", w13), ("w13_scale", w13_scale), ("w2", w2), ("w2_scale", w2_scale)):
            self.register_buffer(name, t)
        self.register_buffer("bias", bias)
        for i, name in enumerate(("shared_w13", "shared_w13_scale", "shared_w2", "shared_w2_scale")):
            self.register_buffer(name, None if shared is None else shared[i])
        self.top_k, self.mode = top_k, mode
        self.n_groups, self.topk_groups, self.renorm, self.scale = n_groups, topk_groups, renorm, scale
        self._impl = None

    def _moe(self):
        m = self._impl
        if m is None or m.w13.data_ptr() != self.w13.data_ptr():          # built late: `.to(device)` replaces the buffers
            shared = None if self.shared_w13 is None else (self.shared_w13, self.shared_w13_scale, self.shared_w2,
                                                           self.shared_w2_scale)
            m = self._impl = FusedMoE(self.router_weight, self.w13, self.w13_scale, self.w2, self.w2_scale, self.top_k,
                                      self.mode, self.bias, self.n_groups, self.topk_groups, self.renorm, self.scale, shared)
        return m

    @torch.no_grad()
    def forward(self, x):
        return self._moe()(x)
