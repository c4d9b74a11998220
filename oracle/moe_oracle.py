"""CPU oracle for the FP8 fused-MoE inference path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module: it is
the checker that the parity tests, the smoke test and the benchmark's CPU-baseline
leg compare the HIP path against.  It restates, in plain torch-CPU / numpy, the CPU
ground truth that the reference keeps inside its own tests, plus the closed-form
definitions of the pieces the reference leaves to closed-source code.

What follows which reference lines (paths relative to the reference root):

  weight_dequant_literal      python/regression/test_llm/test_moe.py:10-50
  dequant_block               same arithmetic, vectorised (fusedMoE.pl:11-34)
  mlp_ref_bf16 / experts_ref_bf16
                              python/regression/test_llm/test_moe.py:63-98
                              (bf16 chain because of set_default_dtype at :261)
  cos_sim / cal_diff          torch_tpu/utils/compare.py:5-22
  noaux_tc_topk               python/regression/test_llm/test_noaux_tc_topk.py:10-37
  route_sigmoid_recipe        python/regression/test_llm/test_torch_ops.py:441-456
  permute_literal             torch_tpu/csrc/ops/my_ops/fusedMoE.pl:624-756
  permute_counting_sort       the same permutation as a stable counting sort
  mlp_w8a16_dq_ref            python/regression/test_llm/test_mlp_w8a16_dq.py:53-81
  mm_w8a16_dq_ref             python/regression/test_llm/test_mm_w8a16_dq.py:52-60

Pinned by tests/test_oracle.py against: the reference's routing tables and its
``err_data`` vector (tests/golden/reference_fixtures.json), brute force on tiny
inputs, library routines (torch.sort / torch.topk on distinct values / bincount /
F.linear) and closed forms (all 256 e4m3fn codes, scale==1 dequant, E=1 MoE ==
dense MLP).

Parity unpinned (the reference holds no source, test or vector for them; they are
defined here from the workload description and closed forms only):
  act_quant_group128, quant_weight_block128, experts_w8a8_fp32, moe_w8a8_fp32,
  mlp_w8a8_fp32, mm_w8a8_fp32, route_softmax_topk, route_sigmoid_grouped (bias handling).
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

FP8_MAX = 448.0          # largest finite OCP e4m3fn magnitude
BLOCK = 128              # weight block edge and activation group width
ACT_EPS = 1e-10          # floor on a group's amax before it becomes a scale


# --------------------------------------------------------------------------- #
# e4m3fn, written out independently of torch's cast so the cast can be pinned
# --------------------------------------------------------------------------- #
def e4m3_decode_table() -> np.ndarray:
    """Value of each of the 256 OCP e4m3fn codes (bias 7, no inf, 0x7f/0xff NaN)."""
    out = np.zeros(256, dtype=np.float32)
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            v = float("nan")
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[c] = -v if s else v
    return out


def e4m3_encode_np(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even encode of float32 values with |x| <= 448 (brute force
    nearest-code search; ties go to the even code)."""
    x = np.asarray(x, dtype=np.float32)
    tab = e4m3_decode_table()[:0x7F].astype(np.float64)       # 0 .. 448 ascending
    a = np.abs(x).astype(np.float64)
    hi = np.clip(np.searchsorted(tab, a, side="left"), 0, 0x7E)
    lo = np.clip(hi - 1, 0, 0x7E)
    dlo, dhi = np.abs(a - tab[lo]), np.abs(tab[hi] - a)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    return code | (np.signbit(x).astype(np.uint8) << 7)


def to_e4m3(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> e4m3fn with saturation at +-448 (torch's cast alone turns >464 into NaN)."""
    return x.float().clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


# --------------------------------------------------------------------------- #
# block-scaled weights
# --------------------------------------------------------------------------- #
def weight_dequant_literal(x: torch.Tensor, s: torch.Tensor, block_size: int = BLOCK,
                           out_dtype=torch.bfloat16) -> torch.Tensor:
    """Block loop exactly as the reference's test helper does it: each block is
    ``fp8.to(fp32) * s[i, j]`` and is stored in ``out_dtype`` (bf16 in the reference,
    whose tests switch the default dtype)."""
    assert x.dim() == 2 and s.dim() == 2
    M, N = x.shape
    y = torch.empty(M, N, dtype=out_dtype)
    for bi in range((M + block_size - 1) // block_size):
        for bj in range((N + block_size - 1) // block_size):
            r0, r1 = bi * block_size, min((bi + 1) * block_size, M)
            c0, c1 = bj * block_size, min((bj + 1) * block_size, N)
            y[r0:r1, c0:c1] = x[r0:r1, c0:c1].to(torch.float32) * s[bi, bj]
    return y


def expand_block_scale(s: torch.Tensor, rows: int, cols: int, block: int = BLOCK) -> torch.Tensor:
    return s.repeat_interleave(block, -2).repeat_interleave(block, -1)[..., :rows, :cols]


def dequant_block(q: torch.Tensor, s: torch.Tensor, block: int = BLOCK,
                  out_dtype=torch.float32) -> torch.Tensor:
    """Vectorised ``q.float() * s[row//block, col//block]`` (ragged edges allowed)."""
    rows, cols = q.shape[-2:]
    return (q.to(torch.float32) * expand_block_scale(s.to(torch.float32), rows, cols, block)).to(out_dtype)


def quant_weight_block128(w: torch.Tensor, block: int = BLOCK):
    """[..., N, K] float weights -> (e4m3fn codes, fp32 scale per block), scale = amax/448."""
    w = w.to(torch.float32)
    N, K = w.shape[-2:]
    nb, kb = -(-N // block), -(-K // block)
    pad = F.pad(w, (0, kb * block - K, 0, nb * block - N))
    blk = pad.reshape(*w.shape[:-2], nb, block, kb, block)
    amax = blk.abs().amax(dim=(-3, -1))
    s = amax.clamp_min(ACT_EPS) / FP8_MAX
    q = to_e4m3(w / expand_block_scale(s, N, K, block))
    return q, s


# --------------------------------------------------------------------------- #
# per-token, per-128-column activation quantisation
# --------------------------------------------------------------------------- #
def act_quant_group128(x: torch.Tensor, group: int = BLOCK):
    """[R, C] -> (e4m3fn [R, C], fp32 scales [R, ceil(C/group)]).
    scale = max(amax, 1e-10) / 448 ; q = clamp(x / scale, +-448) rounded to nearest even."""
    x = x.to(torch.float32)
    R, C = x.shape
    g = -(-C // group)
    pad = F.pad(x, (0, g * group - C)).reshape(R, g, group)
    s = pad.abs().amax(-1).clamp_min(ACT_EPS) / FP8_MAX
    q = to_e4m3(pad / s.unsqueeze(-1)).reshape(R, g * group)[:, :C].contiguous()
    return q, s


def act_dequant_group128(q: torch.Tensor, s: torch.Tensor, group: int = BLOCK) -> torch.Tensor:
    R, C = q.shape
    return q.to(torch.float32) * s.repeat_interleave(group, -1)[:, :C]


# --------------------------------------------------------------------------- #
# routing
# --------------------------------------------------------------------------- #
def topk_lowest_index(scores: torch.Tensor, k: int):
    """top-k along the last dim, values compared in fp32, equal values resolved in
    favour of the lower index (the reference never exercises ties: its inputs are
    permutations).  Returns (values in scores' dtype, int64 indices), descending."""
    order = torch.sort(scores.to(torch.float32), dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.gather(scores, -1, order), order


def noaux_tc_topk(scores: torch.Tensor, n_groups: int, topk_groups: int, top_k: int):
    """DeepSeek-V3 group-limited top-k: group score = sum of the group's two best
    scores (in scores' dtype, as the reference's ground truth computes it), keep the
    ``topk_groups`` best groups, top_k over what is left.  Returns (values, int32 ids)."""
    T, E = scores.shape
    grouped = scores.reshape(T, n_groups, E // n_groups)
    top2 = topk_lowest_index(grouped, 2)[0]
    group_scores = (top2[..., 0].to(torch.float32) + top2[..., 1].to(torch.float32)).to(scores.dtype)
    keep = topk_lowest_index(group_scores, topk_groups)[1]
    mask = torch.ones(T, n_groups, dtype=torch.bool).scatter_(1, keep, False)
    masked = grouped.masked_fill(mask.unsqueeze(-1), float("-inf")).reshape(T, E)
    values, idx = topk_lowest_index(masked, top_k)
    return values, idx.to(torch.int32)


def noaux_tc_topk_bruteforce(row, n_groups, topk_groups, top_k):
    """Same selection for ONE row of distinct python floats, by sorting lists."""
    E = len(row)
    per = E // n_groups
    gs = []
    for g in range(n_groups):
        vals = sorted(row[g * per:(g + 1) * per], reverse=True)
        gs.append((vals[0] + vals[1], -g))
    keep = {-g for _, g in sorted(gs, reverse=True)[:topk_groups]}
    cand = [(row[i], -i) for i in range(E) if i // per in keep]
    best = sorted(cand, reverse=True)[:top_k]
    return [v for v, _ in best], [-i for _, i in best]


def route_softmax_topk(logits: torch.Tensor, k: int, renorm: bool = True):
    """softmax over all experts, top-k (selected on the raw logits: same order),
    optionally renormalised over the selected ones.  -> (fp32 weights, int32 ids)."""
    logits = logits.to(torch.float32)
    _, ids = topk_lowest_index(logits, k)
    p = torch.softmax(logits, dim=-1)
    w = torch.gather(p, -1, ids)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w, ids.to(torch.int32)


def sigmoid_scores(logits: torch.Tensor) -> torch.Tensor:
    return torch.sigmoid(logits.to(torch.float32))


def select_sigmoid_grouped(scores: torch.Tensor, bias, k: int, n_groups: int, topk_groups: int,
                           scale: float = 2.5, renorm: bool = True):
    """Selection half of the sigmoid router, from given fp32 scores: choose on
    ``scores + bias`` with group limiting, weigh with the un-biased scores,
    ``w / sum(w) * scale``.  -> (fp32 weights, int32 ids)."""
    scores = scores.to(torch.float32)
    sel = scores if bias is None else scores + bias.to(torch.float32)
    if n_groups > 1:
        _, ids = noaux_tc_topk(sel, n_groups, topk_groups, k)
    else:
        ids = topk_lowest_index(sel, k)[1].to(torch.int32)
    w = torch.gather(scores, -1, ids.long())
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w * scale, ids


def route_sigmoid_grouped(logits, bias, k, n_groups, topk_groups, scale=2.5, renorm=True):
    return select_sigmoid_grouped(sigmoid_scores(logits), bias, k, n_groups, topk_groups, scale, renorm)


def route_sigmoid_recipe(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int, scale: float = 2.5):
    """The callers' recipe as the reference writes it out with aten ops:
    matmul -> sigmoid -> topk -> sum -> div -> mul."""
    logits = torch.matmul(x, gate_weight.T)
    s = torch.sigmoid(logits)
    w, ids = torch.topk(s, top_k, dim=1)
    return torch.mul(torch.div(w, torch.sum(w, dim=1, keepdim=True)), scale), ids


# --------------------------------------------------------------------------- #
# permutation
# --------------------------------------------------------------------------- #
def permute_literal(select_experts: torch.Tensor, num_experts: int):
    """What the reference kernel's index-building phases produce, by brute force:
    per expert the ascending token ids routed to it (gather side) and the
    ascending flat slot ids t*K+k (scatter side)."""
    T, K = select_experts.shape
    sel = select_experts.tolist()
    gather, scatter = [], []
    for e in range(num_experts):
        gather.append([t for t in range(T) if e in sel[t]])
        scatter.append([t * K + k for t in range(T) for k in range(K) if sel[t][k] == e])
    return gather, scatter


def permute_counting_sort(select_experts: torch.Tensor, num_experts: int):
    """Stable counting sort of the flattened [T*K] expert ids.
    -> sorted_slot int32 [T*K] (flat slot ids grouped by expert, ascending inside an
    expert), expert_offsets int32 [E+1], slot_to_row int32 [T*K] (inverse)."""
    flat = select_experts.reshape(-1).to(torch.int64)
    if flat.numel() and (flat.min() < 0 or flat.max() >= num_experts):
        raise ValueError("expert id out of range")
    sorted_slot = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    slot_to_row = torch.empty_like(sorted_slot)
    slot_to_row[sorted_slot] = torch.arange(flat.numel())
    return sorted_slot.to(torch.int32), offsets.to(torch.int32), slot_to_row.to(torch.int32)


# --------------------------------------------------------------------------- #
# reference-form experts: bf16 activations, fp8 weights with block scales,
# un-weighted per-slot output [T, K, H]
# --------------------------------------------------------------------------- #
def mlp_ref_bf16(x, w0, w1, w2, s0, s1, s2, block=BLOCK):
    """One expert on rows x [n, H] in the reference's bf16 chain.  w0/w1 [I, H],
    w2 [H, I] (HF orientation, as the reference's CPU side keeps it); scales None
    means the weights are already bf16."""
    def deq(w, s):
        return w.to(torch.bfloat16) if s is None else dequant_block(w, s, block, torch.bfloat16)
    x = x.to(torch.bfloat16)
    g = F.silu(F.linear(x, deq(w0, s0)))
    u = F.linear(x, deq(w1, s1))
    return F.linear(g * u, deq(w2, s2))


def experts_ref_bf16_literal(x, select_experts, w0, w1, w2, s0, s1, s2, block=BLOCK):
    """Per (token, slot) loop with the literal block-loop dequant: tiny inputs only."""
    T, K = select_experts.shape
    out = torch.zeros(T, K, x.shape[1], dtype=torch.bfloat16)
    x = x.to(torch.bfloat16)
    for t in range(T):
        for k in range(K):
            e = int(select_experts[t, k])
            d0 = weight_dequant_literal(w0[e], s0[e], block)
            d1 = weight_dequant_literal(w1[e], s1[e], block)
            d2 = weight_dequant_literal(w2[e], s2[e], block)
            h = F.silu(F.linear(x[t], d0)) * F.linear(x[t], d1)
            out[t, k] = F.linear(h, d2)
    return out


def experts_ref_bf16(x, select_experts, w0, w1, w2, s0, s1, s2, block=BLOCK):
    """Same result, one dequant per touched expert."""
    T, K = select_experts.shape
    out = torch.zeros(T * K, x.shape[1], dtype=torch.bfloat16)
    flat = select_experts.reshape(-1).to(torch.int64)
    for e in torch.unique(flat).tolist():
        slots = torch.nonzero(flat == e).squeeze(-1)
        rows = x[slots // K]
        out[slots] = mlp_ref_bf16(rows, w0[e], w1[e], w2[e],
                                  None if s0 is None else s0[e],
                                  None if s1 is None else s1[e],
                                  None if s2 is None else s2[e], block)
    return out.reshape(T, K, -1)


# --------------------------------------------------------------------------- #
# W8A8 pipeline in fp32 on the same quantised operands
# --------------------------------------------------------------------------- #
def experts_w8a8_fp32(x, select_experts, w13q, w13s, w2q, w2s, block=BLOCK, return_mid=False, mid=None):
    """x [T,H] bf16; w13q [E,2I,H] e4m3 (gate rows then up rows), w13s [E,2I/128,H/128]
    fp32; w2q [E,H,I], w2s [E,H/128,I/128].  Every product is taken between
    dequantised fp32 operands; the SwiGLU output is re-quantised per row per 128
    columns before the second GEMM.  -> fp32 [T, K, H] un-weighted.

    mid = (hq uint8 [T,K,I], hs fp32 [T,K,I/128]): use these re-quantised SwiGLU
    outputs instead of computing them (second GEMM only).  The re-quantisation
    rounds values that sit on a rounding boundary either way depending on the
    last bits of the fp32 sum, so two correct implementations of the first GEMM
    can differ by one e4m3 step in isolated elements; this hook lets a test check
    the second GEMM on exactly the operands another implementation produced."""
    T, K = select_experts.shape
    H = x.shape[1]
    I = w2q.shape[2]
    xq, xs = act_quant_group128(x, block)
    xd = act_dequant_group128(xq, xs, block)
    out = torch.zeros(T * K, H, dtype=torch.float32)
    hq_all = torch.zeros(T * K, I, dtype=torch.uint8)
    hs_all = torch.zeros(T * K, -(-I // block), dtype=torch.float32)
    flat = select_experts.reshape(-1).to(torch.int64)
    for e in torch.unique(flat).tolist():
        slots = torch.nonzero(flat == e).squeeze(-1)
        if mid is None:
            rows = xd[slots // K]
            gu = rows @ dequant_block(w13q[e], w13s[e], block).T
            h = F.silu(gu[:, :I]) * gu[:, I:]
            hq, hs = act_quant_group128(h, block)
        else:
            hq = mid[0].reshape(T * K, I)[slots].view(torch.float8_e4m3fn)
            hs = mid[1].reshape(T * K, -1)[slots]
        out[slots] = act_dequant_group128(hq, hs, block) @ dequant_block(w2q[e], w2s[e], block).T
        if return_mid:
            hq_all[slots] = hq.view(torch.uint8)
            hs_all[slots] = hs
    out = out.reshape(T, K, H)
    if return_mid:
        return out, (xq, xs, hq_all.reshape(T, K, I), hs_all.reshape(T, K, -1))
    return out


# --------------------------------------------------------------------------- #
# dense layers (the same arithmetic with one expert that owns every row)
# --------------------------------------------------------------------------- #
def mlp_w8a16_dq_ref(x, gate_weight, up_weight, down_weight, gate_scale, up_scale, down_scale, block=BLOCK):
    """Reference form: block-dequantise each weight into bf16 (block loop), then a bf16
    F.linear / F.silu chain.  gate/up [I, H], down [H, I] in checkpoint orientation."""
    x = x.to(torch.bfloat16)
    g = F.silu(F.linear(x, weight_dequant_literal(gate_weight, gate_scale, block)))
    u = F.linear(x, weight_dequant_literal(up_weight, up_scale, block))
    return F.linear(g * u, weight_dequant_literal(down_weight, down_scale, block))


def mm_w8a16_dq_ref(x, weight, scale, block=BLOCK):
    """Reference form: block-dequantise w [N, K] into bf16, then F.linear in bf16 (ragged N allowed)."""
    return F.linear(x.to(torch.bfloat16), weight_dequant_literal(weight, scale, block))


def mm_w8a8_fp32(x, wq, ws, block=BLOCK):
    """x [M, K] bf16 quantised per row and 128 columns, times dequantised w [N, K]^T, all in fp32."""
    xq, xs = act_quant_group128(x, block)
    return act_dequant_group128(xq, xs, block) @ dequant_block(wq, ws, block).T


def mlp_w8a8_fp32(x, w13q, w13s, w2q, w2s, block=BLOCK, return_mid=False, mid=None):
    """Dense gated MLP on quantised operands: experts_w8a8_fp32 with a single expert and a single
    slot per row.  w13q [2I, H], w2q [H, I]."""
    sel = torch.zeros(x.shape[0], 1, dtype=torch.int32)
    r = experts_w8a8_fp32(x, sel, w13q[None], w13s[None], w2q[None], w2s[None], block, return_mid, mid)
    if return_mid:
        return r[0][:, 0], r[1]
    return r[:, 0]


def e4m3_step(code_u8: torch.Tensor) -> torch.Tensor:
    """Grid spacing of e4m3fn around each code (distance to the next larger magnitude)."""
    mag = (code_u8 & 0x7F).to(torch.int64)
    tab = torch.from_numpy(e4m3_decode_table()[:0x7F].copy())
    up = tab[(mag + 1).clamp(max=0x7E)] - tab[mag.clamp(max=0x7E)]
    down = tab[mag.clamp(max=0x7E)] - tab[(mag - 1).clamp(min=0)]
    return torch.maximum(up, down)


def weighted_reduce(per_slot: torch.Tensor, routing_weights: torch.Tensor) -> torch.Tensor:
    return torch.einsum("tk,tkh->th", routing_weights.to(torch.float32), per_slot.to(torch.float32))


def moe_w8a8_fp32(x, select_experts, routing_weights, w13q, w13s, w2q, w2s, shared=None, block=BLOCK):
    """Routed experts + weighted reduce (+ a shared expert applied to every token
    with weight 1) in fp32.  shared = (w13q, w13s, w2q, w2s) each with leading dim 1."""
    y = weighted_reduce(experts_w8a8_fp32(x, select_experts, w13q, w13s, w2q, w2s, block), routing_weights)
    if shared is not None:
        T = x.shape[0]
        zeros = torch.zeros(T, 1, dtype=torch.int32)
        y = y + experts_w8a8_fp32(x, zeros, *shared, block)[:, 0]
    return y


# --------------------------------------------------------------------------- #
# metrics
# --------------------------------------------------------------------------- #
def cos_sim(a, b) -> float:
    a = np.asarray(a, dtype=np.float64).reshape(-1)
    b = np.asarray(b, dtype=np.float64).reshape(-1)
    denom = np.linalg.norm(a) * np.linalg.norm(b)
    cos = 0.0 if denom == 0 else float(a @ b) / denom
    if math.isnan(cos):
        cos = 0.0
    return 0.5 + 0.5 * cos


def cal_diff(x: torch.Tensor, y: torch.Tensor):
    x, y = x.double(), y.double()
    rmse = ((x - y) * (x - y)).mean().sqrt().item()
    cos_diff = 1 - 2 * (x * y).sum().item() / max((x * x + y * y).sum().item(), 1e-12)
    return cos_diff, rmse, (x - y).abs().max().item()


# --------------------------------------------------------------------------- #
# synthetic workloads
# --------------------------------------------------------------------------- #
def make_layer(E, H, I, seed=0, std=0.02, dtype=torch.bfloat16):
    """Random bf16 weights ~N(0, std) quantised to e4m3fn with fp32 128x128 block
    scales, in the packed orientation (W13 = gate rows then up rows; W2 [E,H,I])."""
    g = torch.Generator().manual_seed(seed)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * std).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * std).to(dtype)
    w13q, w13s = quant_weight_block128(w13)
    w2q, w2s = quant_weight_block128(w2)
    return w13q, w13s, w2q, w2s
