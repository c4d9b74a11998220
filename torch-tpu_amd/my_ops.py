"""Registers the reference's operator names in the `my_ops` namespace, so that callers written
against torch-tpu (`torch.ops.my_ops.fused_moe_fused_experts(...)`, positional arguments, caller
allocated outputs) run unchanged on a ROCm device.

Schemas follow the reference's C++ declarations (torch_tpu/csrc/ops/my_ops/ops.hpp:610-676,
716-722; registered at myOps.cpp:73-77).
"""
from __future__ import annotations

import weakref

import torch

from . import ops
from .layer import _pad_to, pack_expert_weights

_lib = torch.library.Library("my_ops", "DEF")

_EXPERTS_HEAD = ("Tensor(a!) output, Tensor input, Tensor? output_sample, Tensor? input_sample, "
                 "Tensor gate_weights, Tensor up_weights, Tensor down_weights, "
                 "Tensor? gate_scales, Tensor? up_scales, Tensor? down_scales, "
                 "Tensor select_experts, Tensor routing_weights, Tensor? num_select_experts, "
                 "Tensor? select_experts_middle, Tensor? routing_weights_middle, ")
_EXPERTS_TAIL = ("int blocksize, int num_experts, int num_experts_per_tok, bool use_grouped_topk, "
                 "int num_expert_group, int topk_group, Tensor? silu, Tensor? sigmoid, Tensor? m0, "
                 "bool save_mid_res) -> Tensor(a!)")

_lib.define("fused_moe_fused_experts(" + _EXPERTS_HEAD + _EXPERTS_TAIL)
_lib.define("fused_moe_fused_experts_v2(" + _EXPERTS_HEAD + "Tensor? gather_buffer, Tensor? scatter_buffer, "
            + _EXPERTS_TAIL)
_lib.define("noaux_tc_topk(Tensor(a!) values, Tensor(b!) indices, Tensor scores, int n_groups, int topk_groups, "
            "int top_k) -> Tensor(a!)")
_lib.define("fused_moe_grouped_topk(Tensor topk_experts_res, Tensor topk_weights_res_bf16, Tensor left_bf16, "
            "Tensor right_bf16, Tensor topk_weights_res, Tensor left, Tensor right, Tensor max, Tensor matmul_res, "
            "Tensor softmax_res) -> Tensor")

# What the reference leaves to its callers or to closed code, as ops of the same namespace: the router recipe
# (python/regression/test_llm/test_torch_ops.py:440-456), the index building of the expert kernel
# (torch_tpu/csrc/ops/my_ops/fusedMoE.pl:624-756) and the weight re-layout (test_moe.py:285-288).
_lib.define("moe_route(Tensor x, Tensor router_weight, Tensor? bias, str mode, int top_k, int n_group, int topk_group, "
            "float scale, bool renorm) -> (Tensor, Tensor)")
_lib.define("moe_permute(Tensor ids, int num_experts) -> (Tensor, Tensor, Tensor)")
_lib.define("moe_pack_weights(Tensor gate_weights, Tensor up_weights, Tensor down_weights, Tensor gate_scales, "
            "Tensor up_scales, Tensor down_scales) -> (Tensor, Tensor, Tensor, Tensor)")

_lib.define("mlp_w8a16_dq_forward(Tensor input, Tensor gate_weight, Tensor up_weight, Tensor down_weight, "
            "Tensor gate_scale, Tensor up_scale, Tensor down_scale, Tensor(a!) output, int blocksize) -> Tensor(a!)")
_lib.define("mm_w8a16_dq_forward(Tensor input, Tensor weight, Tensor scale, Tensor(a!) output, int blocksize) "
            "-> Tensor(a!)")
_lib.define("mlp_w8a8_quant_forward(Tensor input, Tensor gate_weight, Tensor up_weight, Tensor down_weight, "
            "Tensor gate_scale, Tensor up_scale, Tensor down_scale, Tensor(a!) output, int blocksize) -> Tensor(a!)")

# How quantised expert weights are multiplied.  "w8a8" (default): activations are quantised to FP8 per
# token and 128 columns and the products run on the FP8 matrix path - the path this package is about.
# "w8a16": the reference's own arithmetic (python/regression/test_llm/test_moe.py:10-98; fusedMoE.pl:217-269) - bf16
# activations against weights de-quantised to bf16(float(code) * block scale) IN REGISTERS on the way into the
# matrix instructions, from the same packed FP8 copy the default mode reads (one byte per weight element, nothing
# de-quantised in memory); meets the reference's criterion (cos_diff < 1e-4, test_moe.py:308).  Only block sizes
# that 128 does not divide still go through a bf16 copy de-quantised once.  The dense ops mm_w8a16_dq_forward and
# mlp_w8a16_dq_forward follow the same switch.
_numerics = "w8a8"


def set_expert_numerics(mode: str) -> None:
    global _numerics
    if mode not in ("w8a8", "w8a16"):
        raise ValueError("mode must be 'w8a8' or 'w8a16'")
    _numerics = mode


def _dequant_bf16(w, s, blocksize=128):
    """[E, N, K] fp8 with [E, ceil(N/bs), ceil(K/bs)] scales -> bf16, as the reference's weight_dequant does."""
    E, N, K = w.shape
    full = s.to(torch.bfloat16).repeat_interleave(blocksize, dim=1)[:, :N].repeat_interleave(blocksize, dim=2)[:, :, :K]
    return (w.to(torch.float32) * full.to(torch.float32)).to(torch.bfloat16)


class _DerivedCache:
    """Tensors derived from a caller's weight tensors (packed / de-quantised copies), kept for as long as the
    sources live.

    An entry belongs to the source tensor OBJECTS: it holds weak references to them, is found through their ids, is
    valid only while every reference still resolves to the very tensor handed in and address, version counter, shape,
    stride, dtype and device are what they were, and is dropped by a finaliser the moment one of the sources is
    freed - so new weights that land on a recycled address never meet an old copy, and a model with many layers keeps
    one entry per layer (nothing is evicted by count).  An in-place write through `.data` does not move the version
    counter and cannot be seen from here: call `invalidate_weight_cache()` after such an update (or pack explicitly
    with pack_expert_weights and call torch_tpu_amd.fused_experts_fp8 / FusedMoE).  The derived copy doubles the weight
    memory unless the caller drops the originals."""

    def __init__(self):
        self._entries = {}

    @staticmethod
    def _signature(tensors):
        return tuple((t.data_ptr(), t._version, tuple(t.shape), tuple(t.stride()), t.dtype, t.device) for t in tensors)

    def get(self, tensors, tag, make):
        key = (tag,) + tuple(id(t) for t in tensors)
        entry = self._entries.get(key)
        if entry is not None:
            refs, sig, value = entry
            if all(r() is t for r, t in zip(refs, tensors)) and sig == self._signature(tensors):
                return value
        value = make()
        drop = lambda _ref, k=key, d=self._entries: d.pop(k, None)
        self._entries[key] = ([weakref.ref(t, drop) for t in tensors], self._signature(tensors), value)
        return value

    def clear(self):
        self._entries.clear()

    def __len__(self):
        return len(self._entries)


_weights = _DerivedCache()


def invalidate_weight_cache() -> None:
    """Forget every packed / de-quantised copy made for the drop-in ops (needed after weights were overwritten in place
    through `.data`, which no version counter records)."""
    _weights.clear()


def _dense_packed(key_tensors, make, tag="dense"):
    return _weights.get(tuple(key_tensors), tag, make)


def _packed(gate, up, down, gs, us, ds):
    return _weights.get((gate, up, down, gs, us, ds), "experts", lambda: pack_expert_weights(gate, up, down, gs, us, ds))


# One scratch tensor per (device, stream), grown on demand: the ops allocate nothing once it is large enough.
# Calls that share it are ordered by the stream they were enqueued on.
_scratch: dict = {}


def _workspace(device, nbytes: int):
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = _scratch.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _scratch[key] = ws
    return ws


def _zero_ids(device, rows: int):
    """[rows, 1] int32 zeros (every row selects expert 0), kept per device and grown on demand."""
    key = (device, "zero_ids")
    buf = _scratch.get(key)
    if buf is None or buf.numel() < rows:
        buf = torch.zeros(max(rows, 1024), 1, dtype=torch.int32, device=device)
        _scratch[key] = buf
    return buf[:rows]


def _routing_f32(routing_weights, device):
    """The op's routing weights (bf16 in the reference's callers) as fp32 for the weighted sum, in a buffer that is
    kept per (device, stream) next to the workspace."""
    if routing_weights.dtype == torch.float32 and routing_weights.is_contiguous():
        return routing_weights
    key = (device, torch.cuda.current_stream(device).cuda_stream, "rw")
    buf = _scratch.get(key)
    if buf is None or buf.numel() < routing_weights.numel():
        buf = torch.empty(max(routing_weights.numel(), 4096), dtype=torch.float32, device=device)
        _scratch[key] = buf
    out = buf[:routing_weights.numel()].view(routing_weights.shape)
    out.copy_(routing_weights)
    return out


def _fused_experts(output, input, output_sample, input_sample, gate_weights, up_weights, down_weights,
                   gate_scales, up_scales, down_scales, select_experts, routing_weights, num_select_experts,
                   select_experts_middle, routing_weights_middle, blocksize, num_experts, num_experts_per_tok,
                   use_grouped_topk, num_expert_group, topk_group, silu, sigmoid, m0, save_mid_res):
    if select_experts.dtype != torch.int32:
        raise RuntimeError("select_experts must be int32 dtype")
    if num_select_experts is not None and num_select_experts.dtype != torch.int64:
        raise RuntimeError("num_select_experts must be int64 dtype")
    for name, t in (("output_sample", output_sample), ("input_sample", input_sample),
                    ("num_select_experts", num_select_experts), ("silu", silu), ("sigmoid", sigmoid), ("m0", m0)):
        if t is not None:
            raise RuntimeError(f"{name}: the reference never passes this argument and leaves its meaning "
                               "undefined; it is not supported")
    if save_mid_res:
        raise RuntimeError("save_mid_res is not supported")
    if gate_scales is None and up_scales is None and down_scales is None:
        # un-quantised experts (python/test/fused_moe_bf16.py:113-122): bf16 weights, same op
        for t in (gate_weights, up_weights, down_weights):
            if t.dtype != torch.bfloat16:
                raise RuntimeError("weights without scales must be bfloat16")
        w13, w2 = _dense_packed((gate_weights, up_weights, down_weights),
                                lambda: _pack_bf16(gate_weights, up_weights, down_weights), "bf16")
        if w13.shape[0] != num_experts or select_experts.shape[1] != num_experts_per_tok:
            raise RuntimeError("num_experts / num_experts_per_tok do not match the tensors")
        return _padded_io(output, input, w13.shape[2],
                          lambda o, x: _run_bf16(o, x, w13, w2, select_experts, routing_weights))
    if gate_scales is None or up_scales is None or down_scales is None:
        raise RuntimeError("either all three weight tensors carry block scales or none does")
    if blocksize < 1:
        raise RuntimeError("blocksize must be positive")
    # block sizes that 128 does not divide cannot share a 128-long FP8 dot product: the reference's arithmetic then,
    # on a bf16 copy de-quantised once
    if blocksize % 128:
        w13, w2 = _dense_packed(
            (gate_weights, up_weights, down_weights, gate_scales, up_scales, down_scales),
            lambda: _pack_bf16(_dequant_bf16(gate_weights, gate_scales, blocksize),
                               _dequant_bf16(up_weights, up_scales, blocksize),
                               _dequant_bf16(down_weights, down_scales, blocksize)),
            f"dequant{blocksize}")
        return _padded_io(output, input, w13.shape[2],
                          lambda o, x: _run_bf16(o, x, w13, w2, select_experts, routing_weights))
    if blocksize != 128:
        # a multiple of 128: every 128-block takes the scale of the block it lies in (the same products, exactly)
        I, H = gate_weights.shape[1:]
        scales = (gate_scales, up_scales, down_scales)
        w13, w13s, w2, w2s = _dense_packed(
            (gate_weights, up_weights, down_weights, *scales),
            lambda: pack_expert_weights(gate_weights, up_weights, down_weights,
                                        *(_scales_128(t, blocksize, I, H) for t in scales)), f"experts{blocksize}")
    else:
        w13, w13s, w2, w2s = _packed(gate_weights, up_weights, down_weights, gate_scales, up_scales, down_scales)
    if w13.shape[0] != num_experts or select_experts.shape[1] != num_experts_per_tok:
        raise RuntimeError("num_experts / num_experts_per_tok do not match the tensors")
    rw = _routing_f32(routing_weights, input.device) if output.dim() == 2 else None
    return _padded_io(output, input, w13.shape[2], lambda o, x: _run_packed(o, x, w13, w13s, w2, w2s, select_experts, rw))


def _pack_bf16(gate, up, down_t):
    """bf16 weights in the reference's argument layout (gate, up and transposed down, all [E, I, H]) -> (w13, w2)
    tile-blocked, I and H zero-padded to whole 128-blocks like the FP8 weights (layer.stack_expert_weights)."""
    I, H = gate.shape[-2:]
    Ip, Hp = -(-I // 128) * 128, -(-H // 128) * 128
    return (ops.pack_weights(torch.cat([_pad_to(gate, Ip, Hp), _pad_to(up, Ip, Hp)], dim=1).contiguous()),
            ops.pack_weights(_pad_to(down_t, Ip, Hp).transpose(1, 2).contiguous()))


def _padded_io(output, input, Hp, run):
    """Runs `run(output, input)` on a hidden size padded to Hp.  A ragged hidden size (the packed weights were padded to
    whole 128-blocks with zeros): the activations get zero columns to match - they change no group's maximum and add
    nothing to any sum - and the result's padding columns are dropped."""
    H = input.shape[1]
    if Hp == H:
        return run(output, input)
    padded = torch.empty(*output.shape[:-1], Hp, dtype=output.dtype, device=output.device)
    run(padded, torch.nn.functional.pad(input, (0, Hp - H)))
    output.copy_(padded[..., :H])
    return output


def _run_packed(output, input, w13, w13s, w2, w2s, select_experts, rw):
    T, H = input.shape
    E, I2, _ = w13.shape
    if _numerics == "w8a16":
        ws = _workspace(input.device, ops.fused_experts_bf16_workspace_bytes(T, H, I2 // 2, E, select_experts.shape[1]))
        ops.fused_experts_w8a16(input, w13, w13s, w2, w2s, select_experts, rw, out=output, workspace=ws)
        return output
    ws = _workspace(input.device, ops.fused_experts_workspace_bytes(T, H, I2 // 2, E, select_experts.shape[1]))
    ops.fused_experts_fp8(input, w13, w13s, w2, w2s, select_experts, rw, out=output, workspace=ws)
    return output


def _run_bf16(output, input, w13, w2, select_experts, routing_weights):
    T, H = input.shape
    E, I2, _ = w13.shape
    rw = _routing_f32(routing_weights, input.device) if output.dim() == 2 else None
    ws = _workspace(input.device, ops.fused_experts_bf16_workspace_bytes(T, H, I2 // 2, E, select_experts.shape[1]))
    ops.fused_experts_bf16(input, w13, w2, select_experts, rw, out=output, workspace=ws)
    return output


def _fused_experts_v2(output, input, output_sample, input_sample, gate_weights, up_weights, down_weights,
                      gate_scales, up_scales, down_scales, select_experts, routing_weights, num_select_experts,
                      select_experts_middle, routing_weights_middle, gather_buffer, scatter_buffer, blocksize,
                      num_experts, num_experts_per_tok, use_grouped_topk, num_expert_group, topk_group, silu, sigmoid,
                      m0, save_mid_res):
    # the scratch tensors of the reference's second implementation are accepted and left untouched
    return _fused_experts(output, input, output_sample, input_sample, gate_weights, up_weights, down_weights,
                          gate_scales, up_scales, down_scales, select_experts, routing_weights, num_select_experts,
                          select_experts_middle, routing_weights_middle, blocksize, num_experts, num_experts_per_tok,
                          use_grouped_topk, num_expert_group, topk_group, silu, sigmoid, m0, save_mid_res)


def _grouped_topk(*args):
    raise RuntimeError("fused_moe_grouped_topk: the reference's fused router is closed-source, untested and "
                       "undocumented; use noaux_tc_topk or torch_tpu_amd.moe_route instead")


def _moe_route(x, router_weight, bias, mode, top_k, n_group, topk_group, scale, renorm):
    """Router of one layer: logits = x . router_weight^T (bf16, fp32 sums rounded once), then top-k selection and
    weights -> (fp32 weights [T, top_k], int32 ids [T, top_k]).  mode "softmax" | "sigmoid"; bias [E] fp32 takes part in
    the selection only (a softmax router's bias is added to the logits)."""
    if x.dim() != 2 or router_weight.dim() != 2 or x.shape[1] != router_weight.shape[1]:
        raise RuntimeError("x must be [T, H] and router_weight [E, H]")
    E, H = router_weight.shape
    if x.dtype == torch.bfloat16 and router_weight.dtype == torch.bfloat16 and E <= 256 and H % 128 == 0:
        ws = _workspace(x.device, ops.router_logits_workspace_bytes(x.shape[0], H, E))
        logits = ops.router_logits(x.contiguous(), router_weight.contiguous(), workspace=ws)
    else:
        logits = torch.matmul(x, router_weight.t()).contiguous()
        if logits.dtype not in (torch.float32, torch.bfloat16):
            logits = logits.float()
    if mode == "softmax" and bias is not None:
        logits, bias = (logits.float() + bias), None
    return ops.moe_route(logits, top_k, mode, bias, n_group, topk_group, renorm, scale)


def _moe_permute(ids, num_experts):
    return ops.moe_permute(ids, num_experts)


def _moe_pack_weights(gate_weights, up_weights, down_weights, gate_scales, up_scales, down_scales):
    return pack_expert_weights(gate_weights, up_weights, down_weights, gate_scales, up_scales, down_scales)


def _check_dense(blocksize, *fp8):
    if blocksize < 1:
        raise RuntimeError("blocksize must be positive")
    for t in fp8:
        if t.dtype != torch.float8_e4m3fn:
            raise RuntimeError("weights must be float8_e4m3fn")


def _scales_128(s, blocksize, rows, cols):
    """Block scales of a [rows, cols] matrix at a block size that is a multiple of 128, as fp32 scales of
    128 x 128 blocks: every 128-block takes the scale of the block it lies in (the same products, exactly)."""
    m = blocksize // 128
    s = s.to(torch.float32).repeat_interleave(m, dim=-2).repeat_interleave(m, dim=-1)
    return s[..., :(rows + 127) // 128, :(cols + 127) // 128].contiguous()


def _dequant_any(w, s, blocksize):
    """[N, K] fp8 with [ceil(N/bs), ceil(K/bs)] scales -> bf16(fp8) * bf16 scale in bf16, the reference's
    weight_dequant (python/regression/test_llm/test_mm_w8a16_dq.py:10-49) for any block size."""
    N, K = w.shape
    full = s.to(torch.bfloat16).repeat_interleave(blocksize, dim=0)[:N].repeat_interleave(blocksize, dim=1)[:, :K]
    return (w.to(torch.bfloat16) * full).contiguous()


def _mlp_w8a16_dq_forward(input, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, output,
                          blocksize):
    """torch_tpu/csrc/ops/my_ops/MlpW8A16Dq.cpp:189-241: gate/up [I,H], down passed transposed as
    [I,H] (python/regression/test_llm/test_mlp_w8a16_dq.py:106-109), scales likewise; output [M,H].
    Block sizes that are multiples of 128 run the FP8 kernels on the expanded scales; others run the
    reference's own bf16 arithmetic on weights de-quantised once."""
    return _mlp_forward(input, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, output, blocksize,
                        _numerics, True)


def _mlp_w8a8_quant_forward(input, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, output,
                            blocksize):
    """torch_tpu/csrc/ops/my_ops/MlpW8A8Quant.cpp:12-52: the dense gated MLP with quantised activations, same
    arguments as mlp_w8a16_dq_forward.  Always the FP8-activation arithmetic of this package (per-token scales over
    128 columns), whatever set_expert_numerics says.  The reference's implementation is closed and it holds neither a
    test nor a CPU ground truth for this op, so its activation-quantisation numerics are not pinned by anything: what is
    checked is this package's own definition.  The one script that builds arguments for an op of this kind
    (python/test/deepseek_mlp_quant.py:167-177) hands the down projection over as [H, I] with [H/bs, I/bs] scales; that
    orientation is taken as well as the transposed one of the W8A16 op (told apart by shape; a square layer is read the
    W8A16 way)."""
    I, H = gate_weight.shape
    down_t = not (I != H and tuple(down_weight.shape) == (H, I))
    return _mlp_forward(input, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, output, blocksize,
                        "w8a8", down_t)


def _mlp_forward(input, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, output, blocksize,
                 numerics, down_t):
    """down_t: down_weight and down_scale are given transposed ([I, H] / [I/bs, H/bs])."""
    _check_dense(blocksize, gate_weight, up_weight, down_weight)
    I, H = gate_weight.shape
    orient = "t" if down_t else "n"
    as_t = (lambda t: t) if down_t else (lambda t: t.t())        # to the transposed form the packing below expects
    # I or H that 128 does not divide (the reference de-quantises ceil(n/128) blocks, the last one partial:
    # torch_tpu/csrc/ops/my_ops/MlpW8A16Dq.pl:11-34): the packed weights are padded to whole blocks with zeros, the
    # input's columns likewise, and the padded output's first H columns are the result
    Ip, Hp = -(-I // 128) * 128, -(-H // 128) * 128
    M = input.shape[0]
    x = input.contiguous() if Hp == H else torch.nn.functional.pad(input, (0, Hp - H))
    out = output if Hp == H and output.is_contiguous() else torch.empty(M, Hp, dtype=output.dtype, device=output.device)

    def done():
        if out is not output:
            output.copy_(out[:, :H])
        return output

    if blocksize % 128:
        w13, w2 = _dense_packed(
            (gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale),
            lambda: (ops.pack_weights(torch.cat([_pad_to(_dequant_any(gate_weight, gate_scale, blocksize), Ip, Hp),
                                                 _pad_to(_dequant_any(up_weight, up_scale, blocksize), Ip, Hp)], 0)
                                      .unsqueeze(0).contiguous()),
                     ops.pack_weights(_pad_to(_dequant_any(as_t(down_weight), as_t(down_scale), blocksize), Ip, Hp).t()
                                      .unsqueeze(0).contiguous())),
            f"mlp-dequant{blocksize}{orient}")
        # one expert that every row selects; its per-slot result [M, 1, H] is the output itself
        ws = _workspace(input.device, ops.fused_experts_bf16_workspace_bytes(M, Hp, Ip, 1, 1))
        ops.fused_experts_bf16(x, w13, w2, _zero_ids(input.device, M), None, out=out.view(M, 1, Hp), workspace=ws)
        return done()
    w13, w13s, w2, w2s = _dense_packed(
        (gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale),
        lambda: (ops.pack_weights(torch.cat([_pad_to(gate_weight, Ip, Hp), _pad_to(up_weight, Ip, Hp)], 0).contiguous()),
                 torch.cat([_scales_128(gate_scale, blocksize, I, H), _scales_128(up_scale, blocksize, I, H)], 0).contiguous(),
                 ops.pack_weights(_pad_to(as_t(down_weight), Ip, Hp).t().contiguous()),
                 _scales_128(as_t(down_scale), blocksize, I, H).t().contiguous()),
        f"mlp{blocksize}{orient}")
    if numerics == "w8a16" and Hp <= 16384 and Ip <= 16384:
        # the reference's own arithmetic: one expert that every row selects, weights de-quantised in registers
        ids = _zero_ids(input.device, M)
        ws = _workspace(input.device, ops.fused_experts_bf16_workspace_bytes(M, Hp, Ip, 1, 1))
        ops.fused_experts_w8a16(x, w13.unsqueeze(0), w13s.unsqueeze(0), w2.unsqueeze(0), w2s.unsqueeze(0), ids,
                                None, out=out.view(M, 1, Hp), workspace=ws)
        return done()
    ws = _workspace(input.device, ops.mlp_workspace_bytes(M, Hp, Ip))
    ops.mlp_fp8(x, w13, w13s, w2, w2s, out=out, workspace=ws)
    return done()


def _mm_w8a16_dq_forward(input, weight, scale, output, blocksize):
    """torch_tpu/csrc/ops/my_ops/MmW8A16Dq.cpp:185-228: weight [N,K], scale [ceil(N/bs), ceil(K/bs)], output [M,N].
    Block sizes as in mlp_w8a16_dq_forward."""
    _check_dense(blocksize, weight)
    N, K = weight.shape
    # N that 16 does not divide, K that 128 does not divide: zero rows / zero columns up to the next multiple in the
    # packed weight (the reference's blocks at the edges are partial, torch_tpu/csrc/ops/my_ops/MlpW8A16Dq.pl:11-34),
    # zero columns in the input, and the padded output's first N columns are the result
    Np, Kp = -(-N // 16) * 16, -(-K // 128) * 128
    M = input.shape[0]
    x = input.contiguous() if Kp == K else torch.nn.functional.pad(input, (0, Kp - K))
    out = output if Np == N and output.is_contiguous() else torch.empty(M, Np, dtype=output.dtype, device=output.device)

    def done():
        if out is not output:
            output.copy_(out[:, :N])
        return output

    if blocksize % 128:
        (w,) = _dense_packed((weight, scale),
                             lambda: (ops.pack_weights(_pad_to(_dequant_any(weight, scale, blocksize), Np, Kp).contiguous()),),
                             f"mm-dequant{blocksize}")
        ops.mm_bf16(x, w, out=out)
        return done()
    w, ws = _dense_packed((weight, scale), lambda: (ops.pack_weights(_pad_to(weight, Np, Kp).contiguous()),
                                                     _scales_128(scale, blocksize, N, K)), f"mm{blocksize}")
    if _numerics == "w8a16" and Kp <= 16384:
        ops.mm_w8a16(x, w, ws, out=out)
        return done()
    ops.mm_fp8(x, w, ws, out=out, workspace=_workspace(input.device, ops.mm_workspace_bytes(M, Kp, Np)))
    return done()


_lib.impl("fused_moe_fused_experts", _fused_experts, "CompositeExplicitAutograd")
_lib.impl("mlp_w8a16_dq_forward", _mlp_w8a16_dq_forward, "CompositeExplicitAutograd")
_lib.impl("mlp_w8a8_quant_forward", _mlp_w8a8_quant_forward, "CompositeExplicitAutograd")
_lib.impl("mm_w8a16_dq_forward", _mm_w8a16_dq_forward, "CompositeExplicitAutograd")
_lib.impl("fused_moe_fused_experts_v2", _fused_experts_v2, "CompositeExplicitAutograd")
_lib.impl("noaux_tc_topk", ops.noaux_tc_topk, "CompositeExplicitAutograd")
_lib.impl("fused_moe_grouped_topk", _grouped_topk, "CompositeExplicitAutograd")
_lib.impl("moe_route", _moe_route, "CompositeExplicitAutograd")
_lib.impl("moe_permute", _moe_permute, "CompositeExplicitAutograd")
_lib.impl("moe_pack_weights", _moe_pack_weights, "CompositeExplicitAutograd")
