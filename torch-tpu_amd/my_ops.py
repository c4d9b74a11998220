"""The `my_ops` operator namespace of the reference on a ROCm device, so that callers written against torch-tpu
(`torch.ops.my_ops.fused_moe_fused_experts(...)`, positional arguments, caller allocated outputs) run unchanged.

The reference's own MoE ops - fused_moe_fused_experts, fused_moe_fused_experts_v2, noaux_tc_topk,
fused_moe_grouped_topk - are registered from C++ as the reference registers them (`TORCH_LIBRARY(my_ops, m)` with
function pointers, torch_tpu/csrc/ops/my_ops/myOps.cpp:29-80; signatures torch_tpu/csrc/ops/my_ops/ops.hpp:610-676,
716-722): csrc/my_ops.cpp -> libmy_ops_torch.so, which forwards the common call straight to the C ABI.  This module
loads that library, adds the ops the reference keeps elsewhere or leaves to its callers (the dense W8A16 / W8A8
layers, the router recipe, the index building, the weight re-layout) as a fragment of the same namespace, and
implements the rarer forms of the expert op (bf16 weights, other block sizes, ragged sizes, the W8A16 arithmetic)
that the C++ op hands over to `my_ops::_fused_experts_general`.
"""
from __future__ import annotations

import os

import torch
from torch.multiprocessing.reductions import StorageWeakRef

from . import ops
from .layer import _pad_to, pack_expert_weights

_SHIM = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmy_ops_torch.so")
if not os.path.exists(_SHIM):
    raise ImportError(f"{_SHIM} is missing: build it with `python {os.path.join(os.path.dirname(_SHIM), 'build.py')}` "
                      "(g++ against the torch headers). There is no fallback registration.")
torch.ops.load_library(_SHIM)

_lib = torch.library.Library("my_ops", "FRAGMENT")

_EXPERTS_ARGS = ("Tensor output, Tensor input, Tensor? output_sample, Tensor? input_sample, "
                 "Tensor gate_weights, Tensor up_weights, Tensor down_weights, "
                 "Tensor? gate_scales, Tensor? up_scales, Tensor? down_scales, "
                 "Tensor select_experts, Tensor routing_weights, Tensor? num_select_experts, "
                 "Tensor? select_experts_middle, Tensor? routing_weights_middle, "
                 "int blocksize, int num_experts, int num_experts_per_tok, bool use_grouped_topk, "
                 "int num_expert_group, int topk_group, Tensor? silu, Tensor? sigmoid, Tensor? m0, "
                 "bool save_mid_res) -> Tensor")
# the forms of fused_moe_fused_experts that the C++ op does not run itself (same arguments, same result)
_lib.define("_fused_experts_general(" + _EXPERTS_ARGS)

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
    torch.ops.my_ops._set_expert_numerics(0 if mode == "w8a8" else 1)      # the C++ op runs the default mode only


def _dequant_bf16(w, s, blocksize=128):
    """[E, N, K] fp8 with [E, ceil(N/bs), ceil(K/bs)] scales -> bf16, as the reference's weight_dequant does."""
    E, N, K = w.shape
    full = s.to(torch.bfloat16).repeat_interleave(blocksize, dim=1)[:, :N].repeat_interleave(blocksize, dim=2)[:, :, :K]
    return (w.to(torch.float32) * full.to(torch.float32)).to(torch.bfloat16)


class _DerivedCache:
    """Tensors derived from a caller's weight tensors (packed / de-quantised copies), kept for as long as the
    sources live.

    An entry belongs to the STORAGES of the source tensors, not to the Python objects that wrap them (callers
    re-create those freely: `param.data`, a view made per call, tensors re-wrapped by a framework): it is found through
    storage, offset, shape, stride, dtype and device of every source, is valid while every storage is alive and the
    version counters are what they were, and is dropped - the next time the table is touched - once a storage has
    been freed.  The table holds weak references to the storages, so a freed storage's identity cannot be taken over
    by a new one while its entry exists: new weights never meet an old copy, whatever address they land on, and a
    model with many layers keeps one entry per layer (nothing is evicted by count).  An in-place write through
    `.data` does not move the version counter and cannot be seen from here: call `invalidate_weight_cache()` after
    such an update (or pack explicitly with pack_expert_weights and call torch_tpu_amd.fused_experts_fp8 /
    FusedMoE).  The derived copy doubles the weight memory unless the caller drops the originals."""

    def __init__(self):
        self._entries = {}

    @staticmethod
    def _identity(t):
        return (t.untyped_storage()._cdata, t.storage_offset(), tuple(t.shape), tuple(t.stride()), t.dtype, t.device)

    def _purge(self):
        dead = [k for k, (refs, _, _) in self._entries.items() if any(r.expired() for r in refs)]
        for k in dead:
            del self._entries[k]

    def get(self, tensors, tag, make):
        key = (tag,) + tuple(self._identity(t) for t in tensors)
        versions = tuple(t._version for t in tensors)
        entry = self._entries.get(key)
        if entry is not None:
            refs, seen, value = entry
            if seen == versions and not any(r.expired() for r in refs):
                return value
        self._purge()
        value = make()
        self._entries[key] = ([StorageWeakRef(t.untyped_storage()) for t in tensors], versions, value)
        return value

    def clear(self):
        self._entries.clear()

    def __len__(self):
        self._purge()
        return len(self._entries)


_weights = _DerivedCache()


def invalidate_weight_cache() -> None:
    """Forget every packed / de-quantised copy made for the drop-in ops (needed after weights were overwritten in place
    through `.data`, which no version counter records)."""
    _weights.clear()
    torch.ops.my_ops._invalidate_weight_cache()


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


def _w8a16_in_range(*reduction_lengths):
    """The W8A16 kernels keep a token row's step offsets in 16 bits of bf16 elements: reduction lengths up to 16384.
    Beyond that the selected arithmetic is not available, and no other arithmetic is substituted silently."""
    if any(n > 16384 for n in reduction_lengths):
        raise RuntimeError(f"set_expert_numerics('w8a16') covers reduction lengths up to 16384, got {max(reduction_lengths)}; "
                           "use the default 'w8a8' arithmetic for this layer")


def _run_packed(output, input, w13, w13s, w2, w2s, select_experts, rw):
    T, H = input.shape
    E, I2, _ = w13.shape
    if _numerics == "w8a16":
        _w8a16_in_range(H, I2 // 2)
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


def _moe_route(x, router_weight, bias, mode, top_k, n_group, topk_group, scale, renorm):
    """Router of one layer: logits = x . router_weight^T (bf16, fp32 sums rounded once), then top-k selection and
    weights -> (fp32 weights [T, top_k], int32 ids [T, top_k]).  mode "softmax" | "sigmoid"; bias [E] fp32 takes part in
    the selection only (a softmax router's bias is added to the logits)."""
    if x.dim() != 2 or router_weight.dim() != 2 or x.shape[1] != router_weight.shape[1]:
        raise RuntimeError("x must be [T, H] and router_weight [E, H]")
    E, H = router_weight.shape
    # The product runs in bf16 on the matrix cores (what the reference's recipe computes, test_torch_ops.py:440): a
    # router weight held in another dtype, or a hidden size that 128 does not divide, is brought into that form once
    # per weight tensor (zero columns add nothing), the activations per call.
    Hp = -(-H // 128) * 128
    if router_weight.dtype != torch.bfloat16 or Hp != H or not router_weight.is_contiguous():
        (router_weight,) = _dense_packed(
            (router_weight,), lambda: (torch.nn.functional.pad(router_weight.to(torch.bfloat16), (0, Hp - H)).contiguous(),),
            "router")
    if x.dtype != torch.bfloat16 or Hp != H or not x.is_contiguous():
        x = torch.nn.functional.pad(x.to(torch.bfloat16), (0, Hp - H)).contiguous()
    ws = _workspace(x.device, ops.router_logits_workspace_bytes(x.shape[0], Hp, E))
    logits = ops.router_logits(x, router_weight, workspace=ws)
    if mode == "softmax" and bias is not None:
        mode = "softmax_logit_bias"            # a softmax router's bias is part of the logits; the kernel adds it
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
    if numerics == "w8a16":
        _w8a16_in_range(Hp, Ip)
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
    if _numerics == "w8a16":
        _w8a16_in_range(Kp)
        ops.mm_w8a16(x, w, ws, out=out)
        return done()
    ops.mm_fp8(x, w, ws, out=out, workspace=_workspace(input.device, ops.mm_workspace_bytes(M, Kp, Np)))
    return done()


_lib.impl("_fused_experts_general", _fused_experts, "CompositeExplicitAutograd")
_lib.impl("mlp_w8a16_dq_forward", _mlp_w8a16_dq_forward, "CompositeExplicitAutograd")
_lib.impl("mlp_w8a8_quant_forward", _mlp_w8a8_quant_forward, "CompositeExplicitAutograd")
_lib.impl("mm_w8a16_dq_forward", _mm_w8a16_dq_forward, "CompositeExplicitAutograd")
_lib.impl("moe_route", _moe_route, "CompositeExplicitAutograd")
_lib.impl("moe_permute", _moe_permute, "CompositeExplicitAutograd")
_lib.impl("moe_pack_weights", _moe_pack_weights, "CompositeExplicitAutograd")
