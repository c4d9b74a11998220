"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X.

Integer results (routing ids, permutation, e4m3 codes of the activation quantiser) must be
bit-exact; bf16 outputs must be within rtol 2e-2 / atol 1e-2 of the oracle's fp32 computation
on the same quantised operands.
"""
import random

import numpy as np
import pytest
import torch

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-2


def say(*a):
    print(*a, flush=True)


def distinct_ids(T, E, K, seed, gen_weights=True):
    g = torch.Generator().manual_seed(seed)
    ids = torch.argsort(torch.rand(T, E, generator=g), dim=-1)[:, :K].to(torch.int32).contiguous()
    w = torch.rand(T, K, generator=g) + 0.1
    w = (w / w.sum(-1, keepdim=True)).float()
    return ids, w


# ----------------------------------------------------------------------------- quantiser
@pytest.mark.parametrize("R,C", [(1, 128), (16, 256), (33, 7168), (257, 2048)])
def test_act_quant_bit_exact(pkg, oracle, dev, R, C):
    say("act_quant", R, C)
    g = torch.Generator().manual_seed(R * 1000 + C)
    x = torch.randn(R, C, generator=g)
    x[0, :128] = 0.0                                     # an all-zero group
    if R > 1:
        x[1, :128] *= 1e4                                # large magnitudes
        x[1, 128:] *= 1e-6 if C > 128 else 1             # tiny magnitudes
    x = x.to(torch.bfloat16)
    q_ref, s_ref = oracle.act_quant_group128(x)
    q, s = pkg.act_quant(x.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_act_quant_every_value_under_every_scale(pkg, oracle, dev):
    """The quantiser divides by its scale through a refined reciprocal instead of the IEEE division sequence.  Its
    domain is small enough to visit completely: every finite bf16 value x under the scale of every bf16 amax >= |x|
    (a group holds its amax first and 127 candidates after it; candidates above the amax are replaced by zero).
    Codes and scales must equal the oracle's, which divides (oracle/moe_oracle.py: x / scale, round to nearest even)."""
    say("act_quant, exhaustive")
    pos = torch.arange(0, 0x7F80, dtype=torch.int32)                   # +0, denormals, normals up to the largest finite
    vals = torch.cat([pos, pos | 0x8000]).to(torch.int16).view(torch.bfloat16)        # all 65280 finite bf16 values
    n_groups = -(-vals.numel() // 127)
    cand = torch.zeros(n_groups * 127, dtype=torch.bfloat16)
    cand[:vals.numel()] = vals
    cand = cand.view(n_groups, 127)
    cand_abs = cand.float().abs()
    amaxes = pos[1:].to(torch.int16).view(torch.bfloat16)              # every positive finite bf16
    step = 96
    for lo in range(0, amaxes.numel(), step):
        a = amaxes[lo:lo + step]
        x = torch.empty(a.numel(), n_groups, 128, dtype=torch.bfloat16)
        x[:, :, 0] = a[:, None]
        x[:, :, 1:] = torch.where(cand_abs[None] <= a.float()[:, None, None], cand[None], torch.zeros((), dtype=torch.bfloat16))
        x = x.view(-1, 128)
        q, sc = pkg.act_quant(x.to(dev))
        q_ref, s_ref = oracle.act_quant_group128(x)
        assert torch.equal(sc.cpu(), s_ref), lo
        same = q.cpu().view(torch.uint8) == q_ref.view(torch.uint8)
        if not bool(same.all()):
            bad = (~same).nonzero()[0]
            raise AssertionError(f"amax {float(x[bad[0], 0])}: x = {float(x[bad[0], bad[1]])} quantises to "
                                 f"{int(q.cpu().view(torch.uint8)[bad[0], bad[1]])}, the oracle's code is "
                                 f"{int(q_ref.view(torch.uint8)[bad[0], bad[1]])}")


# ----------------------------------------------------------------------------- weight layout
def tile_blocked_reference(w):
    """The tile-blocked byte order written as an index permutation: [tile, row, step, half, chunk, byte] ->
    [tile, step, half, chunk, row, byte] (16-row tiles, 128-byte steps, 16-byte chunks; chunk c of a step sits in
    half c // 4 at position c % 4)."""
    N, K = w.shape[-2:]
    b = w.contiguous().view(torch.uint8).reshape(-1, N // 16, 16, K * w.element_size() // 128, 2, 4, 16)
    return b.permute(0, 1, 3, 4, 5, 2, 6).contiguous().reshape(-1).view(w.dtype).reshape(w.shape)


@pytest.mark.parametrize("shape,dtype", [((16, 128), torch.uint8), ((3, 32, 256), torch.float8_e4m3fn),
                                         ((2, 48, 384), torch.bfloat16), ((5, 1024, 7168), torch.float8_e4m3fn),
                                         ((1536, 7168), torch.float8_e4m3fn)])
def test_pack_weights_is_the_documented_permutation(pkg, dev, shape, dtype):
    say("pack weights", shape, dtype)
    g = torch.Generator().manual_seed(sum(shape))
    raw = torch.randint(0, 256, (*shape[:-1], shape[-1] * torch.empty(0, dtype=dtype).element_size()), generator=g,
                        dtype=torch.uint8)
    w = raw.view(dtype).reshape(shape)
    packed = pkg.pack_weights(w.to(dev))
    torch.cuda.synchronize()
    assert packed.shape == w.shape and packed.dtype == w.dtype
    assert torch.equal(packed.cpu().view(torch.uint8), tile_blocked_reference(w).view(torch.uint8))
    back = pkg.unpack_weights(packed)
    torch.cuda.synchronize()
    assert torch.equal(back.cpu().view(torch.uint8), w.view(torch.uint8))
    # lane l of the first instruction of tile 0, step 0 gets row l % 16, bytes 16 * (l // 16) .. + 15
    flat = packed.cpu().view(torch.uint8).reshape(-1)
    rows = w.view(torch.uint8).reshape(-1, raw.shape[-1])
    for l in (0, 1, 17, 63):
        assert torch.equal(flat[16 * l:16 * l + 16], rows[l % 16, 16 * (l // 16):16 * (l // 16) + 16])
        assert torch.equal(flat[1024 + 16 * l:1024 + 16 * l + 16], rows[l % 16, 64 + 16 * (l // 16):64 + 16 * (l // 16) + 16])


def test_pack_weights_rejects_what_it_cannot_tile(pkg, dev):
    say("pack weights errors")
    with pytest.raises(RuntimeError):
        pkg.pack_weights(torch.zeros(8, 128, dtype=torch.uint8, device=dev))           # rows not a multiple of 16
    with pytest.raises(RuntimeError):
        pkg.pack_weights(torch.zeros(16, 64, dtype=torch.uint8, device=dev))           # a row shorter than a step
    with pytest.raises(RuntimeError):
        pkg.pack_weights(torch.zeros(16, 128, dtype=torch.uint8))                      # not on the GPU
    lib = pkg._lib.lib
    buf = torch.zeros(16, 128, dtype=torch.uint8, device=dev)
    assert lib.moe_pack_weights(None, buf.data_ptr(), 16, 128, buf.data_ptr()) == -5   # in place
    assert lib.moe_pack_weights(None, None, 0, 128, None) == 0                         # nothing to do


# ----------------------------------------------------------------------------- routing
@pytest.mark.parametrize("batch", [1, 8, 16, 64, 128])
def test_noaux_tc_topk_reference_cases(pkg, oracle, dev, batch):
    say("noaux reference case", batch)
    torch.manual_seed(42)
    scores = torch.stack([torch.randperm(256, dtype=torch.float32)]).reshape(1, -1).to(torch.bfloat16).repeat(batch, 1)
    v_ref, i_ref = oracle.noaux_tc_topk(scores.clone(), 8, 4, 8)
    values = torch.empty(batch, 8, dtype=torch.bfloat16, device=dev)
    indices = torch.empty(batch, 8, dtype=torch.int32, device=dev)
    ret = torch.ops.my_ops.noaux_tc_topk(values, indices, scores.to(dev), 8, 4, 8)
    torch.cuda.synchronize()
    assert ret.data_ptr() == values.data_ptr()
    assert torch.equal(indices.cpu(), i_ref)
    assert torch.allclose(values.cpu().float(), v_ref.float(), rtol=1e-5, atol=1e-6)
    assert all(len({i // 32 for i in row}) <= 4 for row in indices.cpu().tolist())


def test_noaux_tc_topk_err_data(pkg, oracle, dev, ref_fixtures):
    say("noaux err_data")
    row = ref_fixtures["noaux_tc_topk_err_data"]
    for dtype in (torch.float32, torch.bfloat16):
        scores = torch.tensor([row], dtype=torch.float32).to(dtype)
        v_ref, i_ref = oracle.noaux_tc_topk(scores, 8, 4, 8)
        values = torch.empty(1, 8, dtype=dtype, device=dev)
        indices = torch.empty(1, 8, dtype=torch.int32, device=dev)
        pkg.noaux_tc_topk(values, indices, scores.to(dev), 8, 4, 8)
        torch.cuda.synchronize()
        assert torch.equal(indices.cpu(), i_ref) and torch.equal(values.cpu(), v_ref)


@pytest.mark.parametrize("T,E,G,TG,K,dtype", [
    (300, 256, 8, 4, 8, torch.float32), (300, 256, 8, 4, 8, torch.bfloat16), (64, 64, 4, 2, 6, torch.float32),
    (17, 16, 8, 3, 2, torch.float32), (5, 1024, 16, 5, 32, torch.float32), (40, 128, 1, 1, 8, torch.float32),
    (9, 96, 3, 2, 7, torch.bfloat16),
])
def test_noaux_tc_topk_random_with_ties(pkg, oracle, dev, T, E, G, TG, K, dtype):
    say("noaux random", T, E, G, TG, K, dtype)
    g = torch.Generator().manual_seed(T + E)
    scores = torch.randn(T, E, generator=g)
    scores[::3] = torch.round(scores[::3] * 2) / 2          # many exact ties
    scores = scores.to(dtype)
    v_ref, i_ref = oracle.noaux_tc_topk(scores, G, TG, K)
    values = torch.empty(T, K, dtype=dtype, device=dev)
    indices = torch.empty(T, K, dtype=torch.int32, device=dev)
    pkg.noaux_tc_topk(values, indices, scores.to(dev), G, TG, K)
    torch.cuda.synchronize()
    assert torch.equal(indices.cpu(), i_ref)
    assert torch.equal(values.cpu(), v_ref)


@pytest.mark.parametrize("T,E,K", [(16, 8, 2), (4096, 8, 2), (1000, 128, 8), (7, 64, 6)])
def test_route_softmax(pkg, oracle, dev, T, E, K):
    say("route softmax", T, E, K)
    g = torch.Generator().manual_seed(E * 7 + T)
    logits = torch.randn(T, E, generator=g) * 2
    w_ref, i_ref = oracle.route_softmax_topk(logits, K, renorm=True)
    w, ids, scores = pkg.moe_route(logits.to(dev), K, "softmax", return_scores=True)
    torch.cuda.synchronize()
    assert torch.equal(ids.cpu(), i_ref)
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    assert torch.allclose(scores.cpu(), torch.softmax(logits, -1), rtol=1e-5, atol=1e-8)
    w2, ids2 = pkg.moe_route(logits.to(dev), K, "softmax", renorm=False)
    w2_ref, _ = oracle.route_softmax_topk(logits, K, renorm=False)
    assert torch.equal(ids2.cpu(), i_ref) and torch.allclose(w2.cpu(), w2_ref, rtol=1e-5, atol=1e-8)
    # bf16 logits are widened exactly
    wb, idb = pkg.moe_route(logits.to(torch.bfloat16).to(dev), K, "softmax")
    wb_ref, idb_ref = oracle.route_softmax_topk(logits.to(torch.bfloat16), K)
    assert torch.equal(idb.cpu(), idb_ref) and torch.allclose(wb.cpu(), wb_ref, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("T,E,K,G,TG,with_bias", [(4096, 256, 8, 8, 4, True), (32, 256, 8, 8, 4, False),
                                                  (16, 128, 4, 1, 1, False), (100, 64, 6, 4, 2, True)])
def test_route_sigmoid_grouped(pkg, oracle, dev, T, E, K, G, TG, with_bias):
    say("route sigmoid", T, E, K, G, TG, with_bias)
    g = torch.Generator().manual_seed(E + T)
    logits = torch.randn(T, E, generator=g)
    bias = (torch.randn(E, generator=g) * 0.1) if with_bias else None
    w, ids, scores = pkg.moe_route(logits.to(dev), K, "sigmoid", bias=None if bias is None else bias.to(dev),
                                   n_groups=G, topk_groups=TG, renorm=True, scale=2.5, return_scores=True)
    torch.cuda.synchronize()
    scores = scores.cpu()
    assert torch.allclose(scores, torch.sigmoid(logits), rtol=1e-6, atol=1e-7)
    # selection is exact GIVEN the scores the device computed (sigmoid may differ in the last ulp)
    w_ref, i_ref = oracle.select_sigmoid_grouped(scores, bias, K, G, TG, 2.5, True)
    assert torch.equal(ids.cpu(), i_ref)
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    # and identical when the same scores are handed in directly
    w3, ids3 = pkg.moe_route(scores.to(dev), K, "scores", bias=None if bias is None else bias.to(dev), n_groups=G,
                             topk_groups=TG, renorm=True, scale=2.5)
    assert torch.equal(ids3.cpu(), i_ref) and torch.allclose(w3.cpu(), w_ref, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("seed", range(30))
def test_routing_random_cases(pkg, oracle, dev, seed):
    """noaux_tc_topk and moe_route on group structures, expert counts, batch sizes (either side of the small-batch
    kernel) and dtypes drawn from the seed, half of them with many exact ties: ids bit-exact against the oracle (lowest
    index wins a tie), values and weights as the oracle's."""
    r = random.Random(3000 + seed)
    G = r.choice([1, 1, 2, 3, 4, 8, 16])
    per = r.choice([2, 3, 4, 7, 16, 32, 64])
    E = G * per if G > 1 else r.choice([2, 3, 8, 17, 64, 100, 256, 1024])
    while E > 1024:
        per //= 2
        E = G * per
    per = E // G
    TG = r.randint(1, G)
    K = r.randint(1, min(32, TG * per))
    T = r.choice([1, 2, 7, 33, 64, 65, 150, 1000])
    dtype = r.choice([torch.float32, torch.bfloat16])
    say("routing random", seed, (T, E, G, TG, K), dtype)
    g = torch.Generator().manual_seed(seed)
    scores = torch.randn(T, E, generator=g)
    if seed % 2:
        scores = torch.round(scores * 2) / 2
    scores = scores.to(dtype)
    v_ref, i_ref = oracle.noaux_tc_topk(scores, G, TG, K)
    values = torch.empty(T, K, dtype=dtype, device=dev)
    indices = torch.empty(T, K, dtype=torch.int32, device=dev)
    pkg.noaux_tc_topk(values, indices, scores.to(dev), G, TG, K)
    torch.cuda.synchronize()
    assert torch.equal(indices.cpu(), i_ref) and torch.equal(values.cpu(), v_ref)
    # the router recipe on the same numbers as logits
    bias = (torch.randn(E, generator=g) * 0.1) if r.random() < 0.5 else None
    bd = None if bias is None else bias.to(dev)
    w, ids, sc = pkg.moe_route(scores.to(dev), K, "sigmoid", bias=bd, n_groups=G, topk_groups=TG, renorm=True, scale=2.5,
                               return_scores=True)
    torch.cuda.synchronize()
    w_ref, ids_ref = oracle.select_sigmoid_grouped(sc.cpu(), bias, K, G, TG, 2.5, True)
    assert torch.equal(ids.cpu(), ids_ref)
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ws, ids_s = pkg.moe_route(scores.to(dev), K, "softmax", renorm=bool(seed % 3))
    ws_ref, ids_s_ref = oracle.route_softmax_topk(scores, K, renorm=bool(seed % 3))
    assert torch.equal(ids_s.cpu(), ids_s_ref)
    assert torch.allclose(ws.cpu(), ws_ref, rtol=1e-5, atol=1e-7)


# ----------------------------------------------------------------------------- permutation
def check_permutation(pkg, oracle, dev, sel, E):
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(sel, E)
    ss, off, s2r = pkg.moe_permute(sel.to(dev), E)
    torch.cuda.synchronize()
    assert torch.equal(off.cpu(), off_ref)
    assert torch.equal(ss.cpu(), ss_ref)
    assert torch.equal(s2r.cpu(), s2r_ref)


@pytest.mark.parametrize("name", ["SELECTED_EXPERTS_B8_E256", "SELECTED_EXPERTS_B22_E256"])
def test_permutation_reference_tables(pkg, oracle, dev, ref_fixtures, name):
    say("permute table", name)
    sel = torch.tensor(ref_fixtures[name], dtype=torch.int32)
    check_permutation(pkg, oracle, dev, sel, 256)
    gather, scatter = oracle.permute_literal(sel, 256)
    ss, off, _ = pkg.moe_permute(sel.to(dev), 256)
    ss, off = ss.cpu(), off.cpu()
    for e in range(256):
        assert ss[off[e]:off[e + 1]].tolist() == scatter[e]


@pytest.mark.parametrize("T,E,K", [(1, 1, 1), (1, 256, 8), (32, 256, 8), (33, 8, 2), (4096, 256, 8), (1000, 1024, 32),
                                   (5000, 3, 2), (16384, 128, 8),
                                   # more than 512 chunks of 256 slots: the scan walks them in more than one round
                                   (30000, 7, 7), (70000, 1000, 2)])
def test_permutation_random(pkg, oracle, dev, T, E, K):
    say("permute random", T, E, K)
    sel, _ = distinct_ids(T, E, K, seed=T + E + K)
    check_permutation(pkg, oracle, dev, sel, E)


def test_permutation_skewed_with_empty_experts(pkg, oracle, dev):
    say("permute zipf")
    T, E, K = 16384, 128, 8
    g = torch.Generator().manual_seed(5)
    bias = -1.2 * torch.log(torch.arange(1, E + 1).float())
    bias[torch.randperm(E, generator=g)[:13]] = -1e9
    logits = torch.randn(T, E, generator=g) + bias
    _, sel = oracle.route_softmax_topk(logits, K)
    counts = torch.bincount(sel.flatten().long(), minlength=E)
    assert (counts == 0).sum() >= 13
    check_permutation(pkg, oracle, dev, sel, E)


# ----------------------------------------------------------------------------- experts
# The SwiGLU output is re-quantised to e4m3 between the two GEMMs.  The FP8 matrix
# instruction sums a 128-long dot product with roughly 2^-12 of its largest product as internal
# error (measured on gfx950), so the device's fp32 sums differ from the oracle's in the last
# ~4 digits and an element sitting on a rounding boundary can land on the neighbouring e4m3
# code.  One such step in a large element moves a whole output row by more than atol.  The
# checks below therefore prove parity in two strict steps plus one end-to-end figure:
#   (1) first GEMM + SwiGLU + re-quantisation: every device code is within one e4m3 step of
#       the oracle's (plus the sums' absolute error for near-zero elements), and all but a sliver
#       are identical; scales agree to 5e-4;
#   (2) second GEMM + un-permute (+ weighted reduce): strict rtol 2e-2 / atol 1e-2, ALL
#       elements, against the oracle run on the very codes the device produced;
#   (3) end to end against the oracle's own codes: the share of elements outside
#       rtol 2e-2 / atol 1e-2 stays below MAX_OUTSIDE and the reference's own metrics hold.
MAX_OUTSIDE = 5e-3


def outside_fraction(got, ref):
    bad = (got - ref).abs() > ATOL + RTOL * ref.abs()
    return bad.float().mean().item()


def check_experts(pkg, oracle, dev, x, layer, ids, w, shared=None):
    T, K = ids.shape
    E, H, I = layer[2].shape
    ref, (xq_ref, xs_ref, hq_ref, hs_ref) = oracle.experts_w8a8_fp32(x, ids, *layer, return_mid=True)
    w13q, w13s, w2q, w2s = pkg.pack_layer(*(t.to(dev) for t in layer))
    xd, idd = x.to(dev), ids.to(dev)

    # ---- staged run through the C ABI
    xq, xs = pkg.act_quant(xd)
    ss, off, s2r, ws = pkg.moe_permute(idd, E, return_workspace=True)
    hq, hs = pkg.gemm1_swiglu(xq, xs, w13q, w13s, (T, K), ss, off, ws)
    y = pkg.gemm2(hq, hs, w2q, w2s, (T, K), ss, off, ws)
    torch.cuda.synchronize()
    assert torch.equal(xq.cpu().view(torch.uint8), xq_ref.view(torch.uint8)) and torch.equal(xs.cpu(), xs_ref)
    ss_ref, off_ref, _ = oracle.permute_counting_sort(ids, E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref)

    # ---- (1) re-quantised SwiGLU output, device rows are in permuted order
    slot = ss.cpu().long()
    hq_dev = torch.empty(T * K, I, dtype=torch.uint8)
    hs_dev = torch.empty(T * K, I // 128, dtype=torch.float32)
    hq_dev[slot] = hq.cpu().view(torch.uint8)
    hs_dev[slot] = hs.cpu()
    hq_r, hs_r = hq_ref.reshape(T * K, I), hs_ref.reshape(T * K, -1)
    # a scale is the largest |h| of 128 columns / 448: it carries the matrix instruction's summation error of that one
    # element (up to 2^-11.8 = 2.8e-4 of the largest product, measured), most visibly where the reduction is short
    assert torch.allclose(hs_dev, hs_r, rtol=5e-4, atol=0)
    v_dev = hq_dev.view(torch.float8_e4m3fn).float()
    v_ref = hq_r.view(torch.float8_e4m3fn).float()
    # one grid step, or (for elements far below the group maximum, where the grid is finer than the
    # fp32 sums' absolute error) 1.4e-4 of the group maximum = 1/16 in units of the scale
    assert ((v_dev - v_ref).abs() <= oracle.e4m3_step(hq_r) + 0.0625).all(), "a code is more than one step off"
    same = (hq_dev == hq_r).float().mean().item()
    assert int((hq_dev != hq_r).sum()) <= 0.005 * hq_dev.numel() + 4, f"only {same:.4f} of the re-quantised codes match"

    # ---- (2) second GEMM on the device's own codes: strict, every element
    y_mid = oracle.experts_w8a8_fp32(x, ids, *layer, mid=(hq_dev.reshape(T, K, I), hs_dev.reshape(T, K, -1)))
    torch.testing.assert_close(y.float().cpu(), y_mid, rtol=RTOL, atol=ATOL)

    # ---- the one-call entry point gives the same bits as the stages
    out = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.fused_experts_fp8(xd, w13q, w13s, w2q, w2s, idd, None, out=out)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16).cpu(), y.view(torch.int16).cpu())
    sh_dev = None if shared is None else pkg.pack_layer(*(t.to(dev) for t in shared))
    out2 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.fused_experts_fp8(xd, w13q, w13s, w2q, w2s, idd, w.to(dev), out=out2, shared=sh_dev)
    torch.cuda.synchronize()
    red_mid = oracle.weighted_reduce(y.float().cpu(), w)        # reduce of the device's bf16 slot results
    red_ref = oracle.weighted_reduce(ref, w)
    if shared is not None:
        sh = oracle.experts_w8a8_fp32(x, torch.zeros(T, 1, dtype=torch.int32), *shared)[:, 0]
        red_mid, red_ref = red_mid + sh, red_ref + sh
        assert outside_fraction(out2.float().cpu(), red_mid) <= MAX_OUTSIDE     # shared path re-quantises too
    else:
        torch.testing.assert_close(out2.float().cpu(), red_mid, rtol=RTOL, atol=ATOL)

    # ---- (3) end to end against the oracle's own intermediate codes
    got = y.float().cpu()
    frac = outside_fraction(got, ref)
    frac2 = outside_fraction(out2.float().cpu(), red_ref)
    cd, _, _ = oracle.cal_diff(ref, got)
    say(f"   codes identical {same:.5f}; outside tolerance: per-slot {frac:.2e}, reduced {frac2:.2e}; cos_diff {cd:.2e}")
    assert frac <= MAX_OUTSIDE and frac2 <= MAX_OUTSIDE
    assert oracle.cos_sim(ref.numpy(), got.numpy()) > 0.9999 and cd < 1e-5
    # the same steps as the full-size tests run them, shared expert included: its re-quantised codes within one step,
    # the final output strict on the device's own codes, the worst end-to-end violation bounded
    rep = entry.load_parity_checks().check_sample(pkg, oracle, xd, idd, (w13q, w13s, w2q, w2s), w_s=w.to(dev),
                                                  shared_dev=sh_dev, y_big=y, out_big=out2, what="experts")
    say(f"   worst violation: per-slot {rep['worst_per_slot']:.2f}, reduced {rep['worst_reduced']:.2f}")
    return got


@pytest.mark.parametrize("T,H,I,E,K", [
    (16, 256, 512, 8, 2),        # the toy configuration
    (1, 256, 128, 1, 1),
    # the reference's grid (python/regression/test_llm/test_moe.py:219-227, 310-316)
    (1, 7168, 256, 1, 1), (1, 7168, 256, 2, 2), (1, 7168, 256, 16, 8), (1, 7168, 256, 256, 8), (8, 7168, 256, 256, 8),
    (17, 512, 384, 8, 2), (33, 512, 256, 4, 2), (64, 1024, 256, 16, 4), (65, 256, 256, 8, 2),
    (200, 512, 256, 8, 2), (300, 256, 128, 3, 2), (256, 7168, 256, 256, 8),
])
def test_fused_experts(pkg, oracle, dev, T, H, I, E, K):
    say("fused experts", T, H, I, E, K)
    layer = oracle.make_layer(E, H, I, seed=H + I + E)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, E, K, seed=T * 3 + E)
    check_experts(pkg, oracle, dev, x, layer, ids, w)


@pytest.mark.parametrize("T,I_sh", [(70, 384), (70, 256), (5, 256), (200, 256)])
def test_fused_experts_with_shared_expert_and_empty_experts(pkg, oracle, dev, T, I_sh):
    """A shared expert of the routed width rides in the routed launches; another width gets its own."""
    say("shared expert", T, I_sh)
    H, I, E, K = 512, 256, 16, 4
    layer = oracle.make_layer(E, H, I, seed=6)
    shared = oracle.make_layer(1, H, I_sh, seed=7)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, 8, K, seed=9)               # experts 8..15 never chosen
    check_experts(pkg, oracle, dev, x, layer, ids, w, shared=shared)


def random_case(seed):
    """A layer shape, a batch size and a routing drawn from the seed: dimensions are multiples of 128 up to 1024, up to 48
    experts, batches from one token to several row tiles of the largest expert, routing uniform or skewed towards a few
    experts (so that one expert holds several row tiles while others stay empty), with or without a shared expert."""
    r = random.Random(seed)
    H, I = 128 * r.randint(1, 8), 128 * r.randint(1, 6)
    E = r.choice([1, 2, 3, 5, 8, 16, 33, 48])
    K = r.randint(1, min(E, 8))
    T = r.choice([1, 2, 7, 15, 16, 17, 31, 33, 63, 64, 65, 100, 129, 257, 400, 650])
    g = torch.Generator().manual_seed(seed)
    skew = r.random() < 0.5
    scores = torch.rand(T, E, generator=g)
    if skew:                       # popularity falls off with the expert's rank; every fifth expert is never chosen
        pop = 1.0 / torch.arange(1, E + 1).float() ** 1.2
        dead = [e for e in range(E) if e % 5 == 4 and E - len(range(4, E, 5)) >= K]
        scores = scores ** (1.0 / pop)
        scores[:, dead] = -1.0
    ids = torch.argsort(scores, dim=-1, descending=True)[:, :K].to(torch.int32).contiguous()
    w = torch.rand(T, K, generator=g) + 0.1
    w = (w / w.sum(-1, keepdim=True)).float()
    I_sh = r.choice([0, 0, I, 128 * r.randint(1, 4)])
    return T, H, I, E, K, ids, w, I_sh


@pytest.mark.parametrize("seed", range(40))
def test_fused_experts_random_shapes(pkg, oracle, dev, seed):
    T, H, I, E, K, ids, w, I_sh = random_case(1000 + seed)
    say("random shape", seed, (T, H, I, E, K), "shared", I_sh, "largest expert",
        int(torch.bincount(ids.flatten().long(), minlength=E).max()))
    assert all(len(set(row.tolist())) == K for row in ids)      # a token's experts are distinct
    layer = oracle.make_layer(E, H, I, seed=seed)
    shared = oracle.make_layer(1, H, I_sh, seed=seed + 77) if I_sh else None
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16)
    check_experts(pkg, oracle, dev, x, layer, ids, w, shared=shared)


def test_my_ops_drop_in_reference_layout(pkg, oracle, dev, checks):
    """The reference's call, argument for argument (python/regression/test_llm/test_moe.py:119-140):
    separate gate/up weights, pre-transposed down, bf16 scales, [T,K,H] output."""
    say("my_ops drop-in")
    T, H, I, E, K = 8, 7168, 256, 256, 8
    g = torch.Generator().manual_seed(1000)
    rnd = random.Random(1000)
    sel = torch.tensor([rnd.sample(range(E), K) for _ in range(T)], dtype=torch.int32)
    w0 = (torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn)
    w1 = (torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn)
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0 = (torch.randn(E, I // 128, H // 128, generator=g) * 0.1).to(torch.bfloat16)
    s1 = (torch.randn(E, I // 128, H // 128, generator=g) * 0.1).to(torch.bfloat16)
    s2 = (torch.randn(E, H // 128, I // 128, generator=g) * 0.1).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    rw = torch.randn(T, K, generator=g).to(torch.bfloat16)
    ref_bf16 = oracle.experts_ref_bf16(x, sel, w0, w1, w2, s0, s1, s2).float()
    ref_w8a8 = oracle.experts_w8a8_fp32(x, sel, torch.cat([w0, w1], 1), torch.cat([s0, s1], 1).float(), w2, s2.float())
    out = torch.empty(T, K, H, dtype=torch.bfloat16, device=dev)
    scratch = [torch.empty(E, T, dtype=torch.int32, device=dev) for _ in range(3)]
    scratch.append(torch.empty(E, T, K, dtype=torch.int32, device=dev))
    args = [out, x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).contiguous().to(dev),
            s0.to(dev), s1.to(dev), s2.transpose(1, 2).contiguous().to(dev), sel.to(dev), rw.to(dev), None]
    tail = [128, E, K, True, 8, 4, None, None, None, False]
    ret = torch.ops.my_ops.fused_moe_fused_experts(*args, scratch[0], scratch[1], *tail)
    torch.cuda.synchronize()
    assert ret.data_ptr() == out.data_ptr()
    got = out.float().cpu()
    scale = ref_w8a8.abs().max().item()
    assert outside_fraction(got / scale, ref_w8a8 / scale) <= MAX_OUTSIDE
    assert oracle.cos_sim(ref_bf16.numpy(), got.numpy()) > 0.99
    # the strict steps on the same call: the op's output rows are the staged kernels' bits on the packed weights
    packed = pkg.pack_expert_weights(w0.to(dev), w1.to(dev), w2.transpose(1, 2).contiguous().to(dev), s0.to(dev), s1.to(dev),
                                     s2.transpose(1, 2).contiguous().to(dev))
    rep = checks.check_sample(pkg, oracle, x.to(dev), sel.to(dev), packed, y_big=out, what="drop-in", unit=scale)
    say("   ", rep)
    out.zero_()
    torch.ops.my_ops.fused_moe_fused_experts_v2(*args, scratch[0], scratch[1], scratch[2], scratch[3], *tail)
    torch.cuda.synchronize()
    assert torch.equal(out.float().cpu(), got)
    # the reference's own arithmetic (weights de-quantised into bf16, bf16 activations) meets the reference's own
    # criterion, cos_sim > 0.99 and cos_diff < 1e-4 (test_moe.py:308)
    pkg.set_expert_numerics("w8a16")
    try:
        out.zero_()
        torch.ops.my_ops.fused_moe_fused_experts(*args, scratch[0], scratch[1], *tail)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got16 = out.float().cpu()
    assert oracle.cos_sim(ref_bf16.numpy(), got16.numpy()) > 0.99
    assert oracle.cal_diff(ref_bf16, got16)[0] < 1e-4


def test_my_ops_registered_from_cpp_keeps_one_packed_copy_per_weight_set(pkg, oracle, dev):
    """The reference's op names come from the C++ extension (TORCH_LIBRARY, function pointers: inferred schemas with
    unnamed arguments).  The packed copy of a weight set belongs to the sources' storages: fresh Python wrappers of the
    same storages (`.data`, views made per call) find it again, an in-place change or new tensors do not; both output
    forms equal the staged entry point on weights packed by hand, bit for bit."""
    say("my_ops C++ registration and its packed-copy table")
    ops = torch.ops.my_ops
    assert ops.fused_moe_fused_experts.default._schema.arguments[0].name == "_0"
    T, H, I, E, K = 5, 512, 256, 8, 2
    g = torch.Generator().manual_seed(77)
    gate, up, down = ((torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn).to(dev) for _ in range(3))
    gs, us, ds = ((torch.rand(E, I // 128, H // 128, generator=g) * 0.1 + 0.01).to(torch.bfloat16).to(dev) for _ in range(3))
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    ids, w = distinct_ids(T, E, K, seed=3)
    ids, w16 = ids.to(dev), w.to(torch.bfloat16).to(dev)
    tail = [None, None, None, 128, E, K, False, 1, 1, None, None, None, False]
    pkg.invalidate_weight_cache()
    assert ops._packed_weight_sets() == 0
    out = torch.empty(T, K, H, dtype=torch.bfloat16, device=dev)
    ops.fused_moe_fused_experts(out, x, None, None, gate, up, down, gs, us, ds, ids, w16, *tail)
    assert ops._packed_weight_sets() == 1
    for _ in range(3):          # new wrapper objects around the same storages: no second copy
        out2 = torch.empty_like(out)
        ops.fused_moe_fused_experts(out2, x, None, None, gate.data, up.view(E, I, H), down[:], gs.data, us.data, ds.data,
                                    ids, w16, *tail)
        assert ops._packed_weight_sets() == 1
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    packed = pkg.pack_expert_weights(gate, up, down, gs, us, ds)
    want = pkg.fused_experts_fp8(x, *packed, ids)
    assert torch.equal(want.view(torch.int16), out.view(torch.int16))
    # the weighted form, routing weights in bf16 as the reference's callers hold them
    red = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    ops.fused_moe_fused_experts(red, x, None, None, gate, up, down, gs, us, ds, ids, w16, *tail)
    want_red = pkg.fused_experts_fp8(x, *packed, ids, w16.float())
    assert torch.equal(red.view(torch.int16), want_red.view(torch.int16))
    # fp32 weights are taken as they are, any other dtype or layout goes through a widened copy: same bits
    for other in (w16.float(), w16.to(torch.float16), w16.t().contiguous().t()):
        red2 = torch.empty_like(red)
        ops.fused_moe_fused_experts(red2, x, None, None, gate, up, down, gs, us, ds, ids, other, *tail)
        assert torch.equal(red2.view(torch.int16), want_red.view(torch.int16)), (other.dtype, other.stride())
    # a recorded in-place change re-packs; so do new tensors
    gs.mul_(2.0)
    ops.fused_moe_fused_experts(out2, x, None, None, gate, up, down, gs, us, ds, ids, w16, *tail)
    assert ops._packed_weight_sets() == 2
    want2 = pkg.fused_experts_fp8(x, *pkg.pack_expert_weights(gate, up, down, gs, us, ds), ids)
    assert torch.equal(out2.view(torch.int16), want2.view(torch.int16))
    del gate
    gate2 = (torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn).to(dev)
    ops.fused_moe_fused_experts(out2, x, None, None, gate2, up, down, gs, us, ds, ids, w16, *tail)
    torch.cuda.synchronize()
    assert ops._packed_weight_sets() == 1          # the entries whose gate storage is gone were dropped on the way
    pkg.invalidate_weight_cache()
    assert ops._packed_weight_sets() == 0
    # enable_profile / disable_profile (torch_tpu/csrc/ops/my_ops/profile.cpp:12-44): GPU time per op between the two
    ops.enable_profile(2, 0)                     # at most two calls recorded, nothing printed
    for _ in range(3):
        ops.fused_moe_fused_experts(out2, x, None, None, gate2, up, down, gs, us, ds, ids, w16, *tail)
    ops.disable_profile()
    report = ops._profile_report()
    line = [l for l in report.splitlines() if l.startswith("fused_moe_fused_experts,")]
    assert len(line) == 1 and int(line[0].split(",")[1]) == 2 and float(line[0].split(",")[2]) > 0.0, report
    ops.fused_moe_fused_experts(out2, x, None, None, gate2, up, down, gs, us, ds, ids, w16, *tail)      # off again
    pkg.invalidate_weight_cache()
    with pytest.raises(RuntimeError, match="do not match"):
        ops.fused_moe_fused_experts(out, x, None, None, gate2, up, down, gs, us, ds, ids, w16, None, None, None, 128, E + 1,
                                    K, False, 1, 1, None, None, None, False)


@pytest.mark.parametrize("block", [64, 256])
@pytest.mark.parametrize("T,H,I,E,K", [(12, 512, 256, 8, 2), (12, 456, 200, 8, 2)])
def test_my_ops_other_block_sizes(pkg, oracle, dev, block, T, H, I, E, K):
    """Block sizes next to 128 (the reference's dense tests use 64 and 256): 256 runs the FP8 kernels on scales
    expanded to 128-blocks, 64 the reference's bf16 arithmetic on weights de-quantised once.  The second shape has
    sizes that no block size divides (partial blocks at the edges, torch_tpu/csrc/ops/my_ops/fusedMoE.pl:11-34)."""
    say("my_ops block", block, T, H, I, E, K)
    g = torch.Generator().manual_seed(block)
    nb = lambda n: (n + block - 1) // block
    sel = torch.argsort(torch.rand(T, E, generator=g), dim=-1)[:, :K].to(torch.int32)
    w0, w1 = ((torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn) for _ in range(2))
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0, s1 = ((torch.rand(E, nb(I), nb(H), generator=g) * 0.1 + 0.01).to(torch.bfloat16) for _ in range(2))
    s2 = (torch.rand(E, nb(H), nb(I), generator=g) * 0.1 + 0.01).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    rw = torch.rand(T, K, generator=g).to(torch.bfloat16)
    ref_bf16 = oracle.experts_ref_bf16(x, sel, w0, w1, w2, s0, s1, s2, block).float()
    out = torch.empty(T, K, H, dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.fused_moe_fused_experts(
        out, x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).contiguous().to(dev), s0.to(dev),
        s1.to(dev), s2.transpose(1, 2).contiguous().to(dev), sel.to(dev), rw.to(dev), None, None, None, block, E, K,
        True, 8, 4, None, None, None, False)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert oracle.cos_sim(ref_bf16.numpy(), got.numpy()) > 0.99
    if block == 64:
        assert oracle.cal_diff(ref_bf16, got)[0] < 1e-4
    elif H % 128 == 0 and I % 128 == 0:
        up = lambda t: t.float().repeat_interleave(2, 1).repeat_interleave(2, 2)
        ref = oracle.experts_w8a8_fp32(x, sel, torch.cat([w0, w1], 1), torch.cat([up(s0), up(s1)], 1), w2, up(s2))
        scale = ref.abs().max().item()
        assert outside_fraction(got / scale, ref / scale) <= MAX_OUTSIDE
    else:
        assert oracle.cal_diff(ref_bf16, got)[0] < 5e-3


def test_layer_module_end_to_end_toy_config(pkg, oracle, dev, checks):
    say("toy config end to end")
    T, H, I, E, K = 16, 256, 512, 8, 2
    layer = oracle.make_layer(E, H, I, seed=0)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    wr = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    layer_dev = pkg.pack_layer(*(t.to(dev) for t in layer))
    moe = pkg.FusedMoE(wr.to(dev), *layer_dev, top_k=K, mode="softmax")
    xd = x.to(dev)
    w, ids = moe.route(xd)
    out = moe.experts(xd, w, ids)
    torch.cuda.synchronize()
    logits_dev = torch.matmul(xd, wr.to(dev).t()).float().cpu()
    w_ref, ids_ref = oracle.route_softmax_topk(logits_dev, K)
    assert torch.equal(ids.cpu(), ids_ref)
    ref = oracle.moe_w8a8_fp32(x, ids_ref, w_ref, *layer)
    assert outside_fraction(out.float().cpu(), ref) <= MAX_OUTSIDE
    checks.check_sample(pkg, oracle, xd, ids, layer_dev, w_s=w, out_big=out, what="toy config")


# ----------------------------------------------------------------------------- full size, graphs
def test_full_size_properties_deepseek_shape(pkg, oracle, dev, checks):
    """DeepSeek-V3 layer shape at T=4096 (too large for the oracle as a whole): routing and permutation
    are checked exactly, the expert output through properties that do not depend on size, and a
    sample of tokens against the oracle."""
    say("full size C3")
    T, H, I, E, K = 4096, 7168, 2048, 256, 8
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    wr = (torch.randn(E, H, generator=g, device=dev) * 0.02).to(torch.bfloat16)

    w13, w13s = pkg.synthetic_weights(E, 2 * I, H, dev, 1)
    w2, w2s = pkg.synthetic_weights(E, H, I, dev, 2)
    logits = torch.matmul(x, wr.t()).float()
    w, ids, scores = pkg.moe_route(logits, K, "sigmoid", None, 8, 4, True, 2.5, return_scores=True)
    w_ref, ids_ref = oracle.select_sigmoid_grouped(scores.cpu(), None, K, 8, 4, 2.5)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5)
    ss, off, s2r = pkg.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids_ref, E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)

    y = pkg.fused_experts_fp8(x, w13, w13s, w2, w2s, ids)                  # [T,K,H]
    out = pkg.fused_experts_fp8(x, w13, w13s, w2, w2s, ids, w)             # [T,H]
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    # (a) the weighted form is the fp32 weighted sum of the per-slot form
    red = torch.einsum("tk,tkh->th", w, y.float())
    torch.testing.assert_close(out.float(), red, rtol=1e-2, atol=1e-2)
    # (b) a token's result does not depend on what else is in the batch, nor on slot order
    sub = torch.arange(0, T, 37, device=dev)
    y_sub = pkg.fused_experts_fp8(x[sub].contiguous(), w13, w13s, w2, w2s, ids[sub].contiguous())
    assert torch.equal(y_sub.view(torch.int16), y[sub].view(torch.int16))
    ids_rev = ids[sub].flip(1).contiguous()
    y_rev = pkg.fused_experts_fp8(x[sub].contiguous(), w13, w13s, w2, w2s, ids_rev)
    assert torch.equal(y_rev.flip(1).view(torch.int16), y[sub].view(torch.int16))
    # (c) eight tokens through the strict steps (codes within one e4m3 step; second GEMM and weighted sum strict
    # on the device's own codes; worst end-to-end violation bounded), their rows of the big batch bit-equal to the
    # staged kernels on those tokens alone
    pick = torch.arange(5, T, 512, device=dev)
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), (w13, w13s, w2, w2s),
                              w_s=w[pick].contiguous(), y_big=y[pick].contiguous(), out_big=out[pick].contiguous(),
                              what="C3 experts")
    say("   ", rep)


def test_hip_graph_replay_matches_eager(pkg, oracle, dev):
    """The whole step under HIP graph capture: replayed several times, with eager work and
    synchronisation in between, every replay must reproduce the eager bits."""
    say("hip graph")
    T, H, I, E, K = 8, 512, 256, 16, 4
    layer = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=21)))
    shared = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(1, H, I, seed=22)))
    g = torch.Generator().manual_seed(23)
    wr = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    moe = pkg.FusedMoE(wr, *layer, top_k=K, mode="sigmoid", n_groups=4, topk_groups=2, scale=2.5, shared=shared)
    xs = [torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev) for _ in range(3)]
    x_static = xs[0].clone()
    out_static = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    eager = [moe(x).clone() for x in xs]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        moe(x_static, out=out_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        moe(x_static, out=out_static)
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_static.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_static, want), f"replay {rep} differs from eager"
            scratch = moe(xs[(rep + 1) % 3])            # eager work between replays
            torch.cuda.synchronize()
            del scratch


def _layer_on_device(pkg, dev, E, H, I, seed):
    return (*pkg.synthetic_weights(E, 2 * I, H, dev, seed), *pkg.synthetic_weights(E, H, I, dev, seed + 1))


def _full_size_checks(pkg, oracle, checks, dev, x, layer, ids, w, pick):
    """Size-independent properties of the expert computation plus a few tokens against the oracle."""
    w13, w13s, w2, w2s = layer
    T = x.shape[0]
    y = pkg.fused_experts_fp8(x, w13, w13s, w2, w2s, ids)
    out = pkg.fused_experts_fp8(x, w13, w13s, w2, w2s, ids, w)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    torch.testing.assert_close(out.float(), torch.einsum("tk,tkh->th", w, y.float()), rtol=1e-2, atol=1e-2)
    sub = torch.arange(0, T, max(1, T // 97), device=dev)
    y_sub = pkg.fused_experts_fp8(x[sub].contiguous(), w13, w13s, w2, w2s, ids[sub].contiguous())
    assert torch.equal(y_sub.view(torch.int16), y[sub].view(torch.int16)), "a token's result depends on the batch"
    y_rev = pkg.fused_experts_fp8(x[sub].contiguous(), w13, w13s, w2, w2s, ids[sub].flip(1).contiguous())
    assert torch.equal(y_rev.flip(1).view(torch.int16), y[sub].view(torch.int16)), "a token's result depends on slot order"
    # the sampled tokens through the strict steps (only the experts they use are brought to the host); their rows of
    # the big batch must be the bits the staged kernels give for those tokens alone
    pick = pick.to(dev)
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), layer, w_s=w[pick].contiguous(),
                              y_big=y[pick].contiguous(), out_big=out[pick].contiguous(), what="full size")
    say("   ", rep)


def test_full_size_properties_mixtral_shape(pkg, oracle, dev, checks):
    """Mixtral-8x7B layer shape (8 experts, top-2, 1024 rows per expert: the matrix-core-bound case) at T=4096."""
    say("full size C2")
    T, H, I, E, K = 4096, 4096, 14336, 8, 2
    layer = _layer_on_device(pkg, dev, E, H, I, 31)
    g = torch.Generator(device=dev).manual_seed(33)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    logits = (torch.randn(T, E, generator=g, device=dev)).float()
    w, ids = pkg.moe_route(logits, K, "softmax", None, 1, 1, True, 1.0)
    w_ref, ids_ref = oracle.route_softmax_topk(logits.cpu(), K, True)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ss, off, s2r = pkg.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids_ref, E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)
    _full_size_checks(pkg, oracle, checks, dev, x, layer, ids, w, torch.tensor([7, 1900, 4095]))
    # the other batch sizes of the same workload (1, 8, 64, 512 tokens: row tiles of 16, 16, 64 and 64/128 rows):
    # the first tokens of the big batch on their own give the same bits, in both output forms
    y = pkg.fused_experts_fp8(x, *layer, ids)
    out = pkg.fused_experts_fp8(x, *layer, ids, w)
    for Ts in (1, 8, 64, 512):
        say("   C2 at T =", Ts)
        xs, ids_s, w_s = x[:Ts].contiguous(), ids[:Ts].contiguous(), w[:Ts].contiguous()
        y_s = pkg.fused_experts_fp8(xs, *layer, ids_s)
        out_s = pkg.fused_experts_fp8(xs, *layer, ids_s, w_s)
        torch.cuda.synchronize()
        assert torch.equal(y_s.view(torch.int16), y[:Ts].view(torch.int16))
        assert torch.equal(out_s.view(torch.int16), out[:Ts].view(torch.int16))


def test_full_size_properties_skewed_load(pkg, oracle, dev, checks):
    """Qwen3-30B-A3B layer shape, T=16384, popularity ~ rank^-1.2 and 13 experts that receive nothing: experts
    with thousands of rows (many row tiles) next to experts with a handful, and empty ones."""
    say("full size C5")
    T, H, I, E, K = 16384, 2048, 768, 128, 8
    layer = _layer_on_device(pkg, dev, E, H, I, 41)
    g = torch.Generator(device=dev).manual_seed(43)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    rank = torch.randperm(E, generator=g, device=dev).float() + 1
    bias = -1.2 * torch.log(rank)
    bias[torch.randperm(E, generator=g, device=dev)[:13]] = -1e9
    logits = torch.randn(T, E, generator=g, device=dev) * 0.9 + bias
    w, ids = pkg.moe_route(logits, K, "softmax", None, 1, 1, True, 1.0)
    w_ref, ids_ref = oracle.route_softmax_topk(logits.cpu(), K, True)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ss, off, s2r = pkg.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids_ref, E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)
    counts = (off_ref[1:] - off_ref[:-1])
    assert int((counts == 0).sum()) >= 13 and int(counts.max()) > 8000
    _full_size_checks(pkg, oracle, checks, dev, x, layer, ids, w, torch.tensor([0, 5000, 11111, 16383]))


# ----------------------------------------------------------------------------- un-quantised experts
@pytest.mark.parametrize("T,H,I,E,K", [(1, 7168, 256, 1, 1), (1, 7168, 256, 16, 8), (1, 7168, 256, 256, 8),
                                       (2, 4096, 384, 2, 2), (8, 4096, 384, 128, 8), (22, 4096, 384, 128, 8),
                                       (300, 512, 256, 8, 2), (2000, 256, 128, 4, 2),
                                       (9, 328, 200, 4, 2), (140, 72, 56, 3, 1)])       # sizes 128 does not divide
def test_experts_with_bf16_weights(pkg, oracle, dev, T, H, I, E, K):
    """The reference's op with the scale arguments absent (python/test/fused_moe_bf16.py:148-208: its shape grid and
    data recipe - everything N(0,1) - plus two larger batches for the big tiles), against the reference's bf16
    chain; its criterion is cos_diff <= 1e-4."""
    say("bf16 experts", T, H, I, E, K)
    g = torch.Generator().manual_seed(1000 + T + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w0 = torch.randn(E, I, H, generator=g).to(torch.bfloat16)
    w1 = torch.randn(E, I, H, generator=g).to(torch.bfloat16)
    w2 = torch.randn(E, H, I, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, E, K, seed=T + 7)
    out = torch.empty(T, K, H, dtype=torch.bfloat16, device=dev)
    r = torch.ops.my_ops.fused_moe_fused_experts(
        out, x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).to(dev), None, None, None,
        ids.to(dev), w.to(torch.bfloat16).to(dev), None, None, None, 128, E, K, False, 1, 1, None, None, None, False)
    torch.cuda.synchronize()
    assert r.data_ptr() == out.data_ptr()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref = oracle.experts_ref_bf16(x, ids, w0, w1, w2, None, None, None).float()
    cos_diff = oracle.cal_diff(ref, got)[0]
    assert cos_diff <= 1e-4, cos_diff
    # element-wise: the chain rounds to bf16 three times (two linears, one product) where the kernel keeps fp32
    # until the intermediate, so a few bf16 steps of the row's scale are allowed
    rms = ref.pow(2).mean().sqrt()
    assert ((got - ref).abs() <= 3e-2 * ref.abs() + 3e-2 * rms).float().mean() > 0.999
    # weighted form
    out2 = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.fused_moe_fused_experts(
        out2, x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).to(dev), None, None, None,
        ids.to(dev), w.to(torch.bfloat16).to(dev), None, None, None, 128, E, K, False, 1, 1, None, None, None, False)
    torch.cuda.synchronize()
    want = torch.einsum("tk,tkh->th", w.to(torch.bfloat16).float(), got)
    rms2 = want.pow(2).mean().sqrt()
    assert ((out2.float().cpu() - want).abs() <= 2e-2 * want.abs() + 2e-2 * rms2).all()


# T x (H, I, E, K) chosen so that every tile height of the grouped kernels runs in this mode: 16, 32 and 64 rows with both
# operands through LDS (and the narrow strips of the second GEMM), 128 and 192 rows with the weights in a register ring
@pytest.mark.parametrize("T,H,I,E,K", [
    (1, 7168, 256, 256, 8), (8, 7168, 256, 256, 8),            # the reference's own shapes (test_moe.py:219-227)
    (16, 512, 256, 8, 2), (30, 512, 384, 8, 2), (64, 1024, 256, 16, 4), (130, 256, 128, 8, 2),
    (128, 768, 128, 64, 2), (260, 512, 256, 8, 2), (600, 512, 256, 4, 2),
])
def test_experts_w8a16_in_registers(pkg, oracle, dev, T, H, I, E, K):
    """The reference's arithmetic on the packed FP8 weights (moe_fused_experts_w8a16): equal, up to the order of the
    matrix instructions' internal sums, to the bf16 kernels on weights de-quantised beforehand by torch,
    bf16(float(code) * scale), and within the reference's own criterion
    (cos_sim > 0.99 and cos_diff < 1e-4, python/regression/test_llm/test_moe.py:308) of the reference's CPU ground
    truth (test_moe.py:10-98) - with nothing de-quantised in memory."""
    say("w8a16 in registers", T, H, I, E, K, "tile", pkg.tile_rows(T, K, E))
    g = torch.Generator().manual_seed(T + H)
    w0, w1 = ((torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn) for _ in range(2))
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0, s1 = ((torch.randn(E, I // 128, H // 128, generator=g) * 0.1).to(torch.bfloat16) for _ in range(2))
    s2 = (torch.randn(E, H // 128, I // 128, generator=g) * 0.1).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, E, K, seed=T + 5)
    w13 = torch.cat([w0, w1], 1).to(dev)
    w13s = torch.cat([s0, s1], 1).float().to(dev)
    w2d, w2s = w2.to(dev), s2.float().to(dev)
    xd, idd, wd = x.to(dev), ids.to(dev), w.to(dev)
    got = pkg.fused_experts_w8a16(xd, pkg.pack_weights(w13), w13s, pkg.pack_weights(w2d), w2s, idd)
    # the same kernels on weights de-quantised in memory
    deq = lambda q, s: (q.float() * s.repeat_interleave(128, 1).repeat_interleave(128, 2)).to(torch.bfloat16)
    want = pkg.fused_experts_bf16(xd, pkg.pack_weights(deq(w13, w13s)), pkg.pack_weights(deq(w2d, w2s)), idd)
    torch.cuda.synchronize()
    # Same weights, same products; the 64 elements of a step sit in other positions of the matrix instructions' reduction
    # (a lane holds 16 consecutive codes here, two runs of 8 bf16 there), and the instruction's internal sum is not
    # associative: fp32 sums differ in the last bits, a few results land on the neighbouring bf16.
    gf, wf = got.float(), want.float()
    same = (got.view(torch.int16) == want.view(torch.int16)).float().mean().item()
    say("    identical to the kernels on weights de-quantised in memory:", same)
    assert same >= 0.97, same
    assert ((gf - wf).abs() <= 1.6e-2 * wf.abs() + 2e-3 * wf.pow(2).mean().sqrt()).all()
    ref = oracle.experts_ref_bf16(x, ids, w0, w1, w2, s0, s1, s2).float()
    got_h = got.float().cpu()
    assert torch.isfinite(got_h).all()
    assert oracle.cos_sim(ref.numpy(), got_h.numpy()) > 0.99
    cos_diff = oracle.cal_diff(ref, got_h)[0]
    assert cos_diff < 1e-4, cos_diff
    # weighted form
    out2 = pkg.fused_experts_w8a16(xd, pkg.pack_weights(w13), w13s, pkg.pack_weights(w2d), w2s, idd, wd)
    want2 = pkg.weighted_reduce(got, wd)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), want2.view(torch.int16))


@pytest.mark.parametrize("T,H,I,E,K", [(9, 320, 192, 8, 2), (70, 448, 200, 4, 2), (3, 7168, 200, 16, 4)])
def test_my_ops_ragged_block_edges(pkg, oracle, dev, T, H, I, E, K):
    """H or I that 128 does not divide: the reference's weight_dequant_bc takes ceil(n/128) blocks, the last one
    partial (torch_tpu/csrc/ops/my_ops/fusedMoE.pl:11-34); here the packed copy is padded to whole blocks with zero
    codes.  Checked against the reference's CPU ground truth on the un-padded tensors (test_moe.py:10-98): the default
    arithmetic within cos_sim > 0.99, the reference's own arithmetic (set_expert_numerics('w8a16')) within its full
    criterion, cos_diff < 1e-4 (test_moe.py:308)."""
    say("ragged", T, H, I, E, K)
    g = torch.Generator().manual_seed(H + I)
    nb = lambda n: (n + 127) // 128
    w0, w1 = ((torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn) for _ in range(2))
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0, s1 = ((torch.randn(E, nb(I), nb(H), generator=g) * 0.1).to(torch.bfloat16) for _ in range(2))
    s2 = (torch.randn(E, nb(H), nb(I), generator=g) * 0.1).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, E, K, seed=T + 11)
    ref = oracle.experts_ref_bf16(x, ids, w0, w1, w2, s0, s1, s2).float()
    args = [x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).contiguous().to(dev),
            s0.to(dev), s1.to(dev), s2.transpose(1, 2).contiguous().to(dev), ids.to(dev), w.to(torch.bfloat16).to(dev), None,
            None, None, 128, E, K, False, 1, 1, None, None, None, False]
    out = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
    r = torch.ops.my_ops.fused_moe_fused_experts(out, *args)
    torch.cuda.synchronize()
    assert r.data_ptr() == out.data_ptr()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert oracle.cos_sim(ref.numpy(), got.numpy()) > 0.99
    assert oracle.cal_diff(ref, got)[0] < 5e-3
    pkg.set_expert_numerics("w8a16")
    try:
        out16 = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
        torch.ops.my_ops.fused_moe_fused_experts(out16, *args)
        out_w = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=dev)
        torch.ops.my_ops.fused_moe_fused_experts(out_w, *args)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got16 = out16.float().cpu()
    assert torch.isfinite(got16).all()
    assert oracle.cos_sim(ref.numpy(), got16.numpy()) > 0.99
    assert oracle.cal_diff(ref, got16)[0] < 1e-4
    want = torch.einsum("tk,tkh->th", w.to(torch.bfloat16).float(), got16)
    assert ((out_w.float().cpu() - want).abs() <= 2e-2 * want.abs() + 2e-2 * want.pow(2).mean().sqrt()).all()


@pytest.mark.parametrize("seed", range(16))
def test_my_ops_random_shapes_both_arithmetics(pkg, oracle, dev, seed):
    """The registered op in the reference's argument layout (python/regression/test_llm/test_moe.py:285-295) on shapes
    drawn from the seed - hidden and intermediate sizes that 128 may or may not divide, one to 64 experts, batches up to
    a few row tiles - through both entry names, against the reference's CPU ground truth (test_moe.py:10-98): the
    reference's own arithmetic within its full criterion (cos_sim > 0.99 and cos_diff < 1e-4, test_moe.py:308), the FP8
    activation path within cos_sim > 0.99, and the [T, H] output form equal to the weighted sum of the [T, K, H] one."""
    r = random.Random(2000 + seed)
    H = r.choice([128 * r.randint(1, 8), 8 * r.randint(9, 120)])
    I = r.choice([128 * r.randint(1, 4), 8 * r.randint(3, 60)])
    E = r.choice([1, 2, 4, 7, 16, 64])
    K = r.randint(1, min(E, 8))
    T = r.choice([1, 3, 8, 17, 40, 96, 200, 330])
    say("my_ops random", seed, (T, H, I, E, K))
    g = torch.Generator().manual_seed(seed)
    nb = lambda n: (n + 127) // 128
    w0, w1 = ((torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn) for _ in range(2))
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0, s1 = ((torch.rand(E, nb(I), nb(H), generator=g) * 0.2 + 0.02).to(torch.bfloat16) for _ in range(2))
    s2 = (torch.rand(E, nb(H), nb(I), generator=g) * 0.2 + 0.02).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids, w = distinct_ids(T, E, K, seed=seed + 3)
    ref = oracle.experts_ref_bf16(x, ids, w0, w1, w2, s0, s1, s2).float()
    wb = w.to(torch.bfloat16)
    args = [x.to(dev), None, None, w0.to(dev), w1.to(dev), w2.transpose(1, 2).contiguous().to(dev),
            s0.to(dev), s1.to(dev), s2.transpose(1, 2).contiguous().to(dev), ids.to(dev), wb.to(dev), None,
            None, None]
    tail = [128, E, K, False, 1, 1, None, None, None, False]
    scratch = [torch.zeros(E, T, dtype=torch.int32, device=dev), torch.zeros(E, T, K, dtype=torch.int32, device=dev)]
    results = {}
    for mode in ("w8a8", "w8a16"):
        pkg.set_expert_numerics(mode)
        try:
            out = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
            torch.ops.my_ops.fused_moe_fused_experts(out, *args, *tail)
            out_v2 = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
            torch.ops.my_ops.fused_moe_fused_experts_v2(out_v2, *args, *scratch, *tail)
            out_w = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=dev)
            torch.ops.my_ops.fused_moe_fused_experts(out_w, *args, *tail)
            torch.cuda.synchronize()
        finally:
            pkg.set_expert_numerics("w8a8")
        assert torch.equal(out.view(torch.int16), out_v2.view(torch.int16)), mode
        got = out.float().cpu()
        assert torch.isfinite(got).all(), mode
        assert oracle.cos_sim(ref.numpy(), got.numpy()) > 0.99, mode
        cd = oracle.cal_diff(ref, got)[0]
        say(f"    {mode}: cos_diff {cd:.2e}")
        assert cd < (1e-4 if mode == "w8a16" else 5e-3), (mode, cd)
        # the [T, H] form: the fp32 weighted sum of the slot results (bf16 routing weights widened), rounded once
        want = torch.einsum("tk,tkh->th", wb.float(), got).to(torch.bfloat16).float()
        gw = out_w.float().cpu()
        assert ((gw - want).abs() <= 1e-2 * want.abs() + 1e-6).all(), mode
        results[mode] = got
