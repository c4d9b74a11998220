"""Pins the CPU oracle: against the reference's own data tables, library routines, closed
forms and brute force.  No GPU, no HIP library."""
import math
import random

import numpy as np
import pytest
import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------- e4m3fn
def test_e4m3_decode_all_codes_match_torch(oracle):
    tab = oracle.e4m3_decode_table()
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(t))
    ok = ~np.isnan(tab)
    assert np.array_equal(tab[ok], t[ok])
    assert tab[0x7E] == 448.0 and tab[0x01] == 2.0 ** -9 and tab[0x38] == 1.0


def test_e4m3_encode_torch_cast_is_rne_after_clamp(oracle):
    tab = oracle.e4m3_decode_table()[:0x7F]
    pts = [tab, -tab]
    mids = 0.5 * (tab[:-1].astype(np.float64) + tab[1:].astype(np.float64))
    mids = mids.astype(np.float32)
    for m in (mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))):
        pts += [m, -m]
    rng = np.random.default_rng(0)
    pts.append(rng.uniform(-448, 448, 100000).astype(np.float32))
    pts.append(rng.uniform(-0.05, 0.05, 100000).astype(np.float32))
    pts.append((rng.standard_normal(100000) * 1000).astype(np.float32))   # exercises the clamp
    x = np.concatenate(pts)
    got = oracle.to_e4m3(torch.from_numpy(x)).view(torch.uint8).numpy()
    want = oracle.e4m3_encode_np(np.clip(x, -448, 448))
    # +0 and -0 codes are both fine for an exact zero result only if they agree in sign handling
    assert np.array_equal(got, want)


def test_e4m3_encode_known_answers(oracle):
    x = np.array([0.0, 1.0, 448.0, 464.0, -448.0, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -9, 0.1], dtype=np.float32)
    want = np.array([0x00, 0x38, 0x7E, 0x7E, 0xFE, 0x00, 0x01, 0x01, 0x1D], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3_encode_np(np.clip(x, -448, 448)), want)


def test_e4m3_step_known_answers_and_closed_form(oracle):
    """e4m3_step sets the tolerance of the 'every re-quantised code within one step' check: pinned against values
    written out by hand and against the format's closed form (three mantissa bits: the grid spacing of a code
    with exponent field e is 2^(max(e,1) - 10); at a binade's lower edge the wider, upper gap counts)."""
    hand = {
        0x00: 2.0 ** -9,       # zero: the smallest subnormal is the next value
        0x03: 2.0 ** -9,       # a subnormal (3 * 2^-9)
        0x07: 2.0 ** -9,       # the largest subnormal, next to the first normal 2^-6
        0x08: 2.0 ** -9,       # first normal 2^-6: both neighbours 2^-9 away
        0x10: 2.0 ** -8,       # binade edge 2^-5: 2^-9 below, 2^-8 above
        0x38: 0.125,           # 1.0: 0.9375 below, 1.125 above
        0x3C: 0.125,           # 1.5
        0x40: 0.25,            # binade edge 2.0: 0.125 below, 0.25 above
        0x77: 16.0,            # 240
        0x78: 32.0,            # binade edge 256
        0x7E: 32.0,            # 448, the largest finite value: 416 below, nothing above
        0xB8: 0.125,           # -1.0: the sign does not matter
        0xFE: 32.0,            # -448
    }
    codes = torch.tensor(sorted(hand), dtype=torch.uint8)
    got = oracle.e4m3_step(codes)
    assert got.dtype == torch.float32
    assert got.tolist() == [hand[int(c)] for c in codes]
    every = torch.tensor([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=torch.uint8)
    closed = torch.tensor([2.0 ** (max((int(c) >> 3) & 15, 1) - 10) for c in every], dtype=torch.float32)
    assert torch.equal(oracle.e4m3_step(every), closed)
    # and it is what the decode table says: the larger of the gaps to the two neighbouring magnitudes
    tab = oracle.e4m3_decode_table()[:0x7F].astype(np.float64)
    for c in (0x01, 0x08, 0x10, 0x38, 0x7D, 0x7E):
        gaps = [tab[c + 1] - tab[c] if c < 0x7E else 0.0, tab[c] - tab[c - 1] if c > 0 else 0.0]
        assert float(oracle.e4m3_step(torch.tensor([c], dtype=torch.uint8))[0]) == max(gaps)
    # shape is kept (the parity checks hand in [rows, I] code matrices)
    assert tuple(oracle.e4m3_step(torch.zeros(3, 5, dtype=torch.uint8)).shape) == (3, 5)


# ----------------------------------------------------------------------------- block dequant
@pytest.mark.parametrize("shape,block", [((256, 384), 128), ((200, 300), 128), ((130, 70), 64), ((300, 520), 256)])
def test_dequant_vectorised_equals_literal_block_loop(oracle, shape, block):
    g = torch.Generator().manual_seed(1)
    q = (torch.randn(*shape, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s = (torch.randn(-(-shape[0] // block), -(-shape[1] // block), generator=g) * 0.1).to(torch.bfloat16)
    lit = oracle.weight_dequant_literal(q, s, block)
    vec = oracle.dequant_block(q, s, block, torch.bfloat16)
    assert torch.equal(lit, vec)
    assert lit.dtype == torch.bfloat16


def test_dequant_unit_scale_is_plain_cast(oracle):
    q = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).reshape(2, 128)
    q = q.view(torch.uint8).clone()
    q[q == 0x7F] = 0
    q[q == 0xFF] = 0
    q = q.view(torch.float8_e4m3fn)
    out = oracle.dequant_block(q, torch.ones(1, 1))
    assert torch.equal(out, q.to(torch.float32))


def test_weight_quant_roundtrip(oracle):
    g = torch.Generator().manual_seed(2)
    w = (torch.randn(3, 256, 384, generator=g) * 0.02).to(torch.bfloat16)
    q, s = oracle.quant_weight_block128(w)
    assert q.dtype == torch.float8_e4m3fn and tuple(s.shape) == (3, 2, 3) and s.dtype == torch.float32
    blk = w.float().reshape(3, 2, 128, 3, 128).abs().amax(dim=(2, 4))
    assert torch.equal(s, blk / 448.0)
    back = oracle.dequant_block(q, s)
    rel = (back - w.float()).abs() / oracle.expand_block_scale(blk, 256, 384)
    assert rel.max() <= 16.0 / 448.0 + 1e-6           # half the grid spacing (32) of the top binade [256, 448]
    # the block maximum itself is hit exactly
    assert torch.equal(back.abs().reshape(3, 2, 128, 3, 128).amax(dim=(2, 4)), blk)


# ----------------------------------------------------------------------------- activation quant
def test_act_quant_closed_form(oracle):
    x = torch.zeros(2, 256)
    x[0, :128] = torch.linspace(-448, 448, 128)          # amax 448 -> scale exactly 1
    x[0, 128:] = 0.0                                     # all-zero group -> eps scale, zero codes
    x[1, 0] = 224.0                                      # amax 224 -> scale 0.5
    x[1, 1] = 0.5
    q, s = oracle.act_quant_group128(x)
    assert s[0, 0].item() == 1.0
    assert s[0, 1].item() == np.float32(1e-10) / np.float32(448.0)
    assert s[1, 0].item() == 0.5
    assert torch.equal(q[0, :128].view(torch.uint8), oracle.to_e4m3(x[0, :128]).view(torch.uint8))
    assert q[0, 128:].view(torch.uint8).abs().sum() == 0
    assert q[1, 0].float().item() == 448.0 and q[1, 1].float().item() == 1.0
    back = oracle.act_dequant_group128(q, s)
    assert back[1, 0].item() == 224.0 and back[1, 1].item() == 0.5


def test_act_quant_error_bound_and_idempotence(oracle):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 512, generator=g).to(torch.bfloat16)
    q, s = oracle.act_quant_group128(x)
    back = oracle.act_dequant_group128(q, s)
    amax = x.float().reshape(64, 4, 128).abs().amax(-1)
    assert torch.equal(s, amax / 448.0)
    err = (back - x.float()).abs().reshape(64, 4, 128)
    assert (err <= amax.unsqueeze(-1) * (16.0 / 448.0) * (1 + 1e-5)).all()   # midpoints hit the bound
    q2, s2 = oracle.act_quant_group128(back)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.allclose(s2, s, rtol=1e-6)


# ----------------------------------------------------------------------------- top-k
def test_topk_lowest_index_matches_torch_on_distinct(oracle):
    g = torch.Generator().manual_seed(4)
    x = torch.stack([torch.randperm(256, generator=g).float() for _ in range(32)]).to(torch.bfloat16)
    v, i = oracle.topk_lowest_index(x, 8)
    tv, ti = torch.topk(x, 8, dim=-1)
    assert torch.equal(v, tv) and torch.equal(i, ti)


def test_topk_lowest_index_ties(oracle):
    x = torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0, 0.0]])
    v, i = oracle.topk_lowest_index(x, 4)
    assert i.tolist() == [[1, 2, 4, 3]] and v.tolist() == [[3.0, 3.0, 3.0, 2.0]]


def _gt_restated(scores, n_groups, topk_groups, top_k):
    """The reference ground truth written with torch.topk (valid when nothing ties)."""
    bs = scores.shape[0]
    sc = scores.clone().view(bs, n_groups, -1)
    group_scores = sc.topk(2, dim=-1)[0].sum(dim=-1)
    idx = group_scores.topk(topk_groups, dim=-1)[1]
    mask = sc.new_ones(bs, n_groups, dtype=torch.bool).scatter_(1, idx, False)
    sc = sc.masked_fill(mask.unsqueeze(-1), float("-inf")).flatten(1)
    return torch.topk(sc, top_k, dim=-1)


def test_noaux_tc_topk_reference_err_data(oracle, ref_fixtures):
    row = ref_fixtures["noaux_tc_topk_err_data"]
    assert sorted(row) == [float(i) for i in range(256)]
    bv, bi = oracle.noaux_tc_topk_bruteforce(row, 8, 4, 8)
    for dtype in (torch.float32, torch.bfloat16):
        scores = torch.tensor([row], dtype=torch.float32).to(dtype)
        v, i = oracle.noaux_tc_topk(scores, 8, 4, 8)
        # in bf16 the group sums are rounded (e.g. 509 -> 508); compare with the brute force run
        # on the same rounding
        if dtype == torch.float32:
            assert i.tolist() == [bi] and v.tolist() == [bv]
        assert len({x // 32 for x in i[0].tolist()}) <= 4
        assert v.dtype == dtype and i.dtype == torch.int32
        assert v[0].float().tolist() == sorted(v[0].float().tolist(), reverse=True)


@pytest.mark.parametrize("batch", [1, 8, 16, 64, 128])
def test_noaux_tc_topk_reference_cases(oracle, batch):
    # the reference's own test input: one seed-42 permutation of 0..255 in bf16, repeated
    torch.manual_seed(42)
    scores = torch.stack([torch.randperm(256, dtype=torch.float32)]).reshape(1, -1).to(torch.bfloat16).repeat(batch, 1)
    v, i = oracle.noaux_tc_topk(scores.clone(), 8, 4, 8)
    gv, gi = _gt_restated(scores, 8, 4, 8)
    assert torch.allclose(gv.float(), v.float(), rtol=1e-5, atol=1e-6)
    assert torch.equal(gi, i.long())
    # brute force in exact arithmetic agrees when the bf16 rounding of the group sums changes no order
    bv, bi = oracle.noaux_tc_topk_bruteforce(scores[0].float().tolist(), 8, 4, 8)
    v32, i32 = oracle.noaux_tc_topk(scores.float(), 8, 4, 8)
    assert i32[0].tolist() == bi


def test_noaux_tc_topk_random_vs_bruteforce(oracle):
    rng = random.Random(5)
    for E, G, TG, K in [(256, 8, 4, 8), (64, 4, 2, 6), (16, 8, 3, 2), (128, 1, 1, 8)]:
        for _ in range(20):
            row = [rng.uniform(-1, 1) for _ in range(E)]
            row32 = torch.tensor([row], dtype=torch.float32)
            bv, bi = oracle.noaux_tc_topk_bruteforce(row32[0].tolist(), G, TG, K)
            if G > 1:
                v, i = oracle.noaux_tc_topk(row32, G, TG, K)
            else:
                v, i = oracle.topk_lowest_index(row32, K)
            assert i[0].tolist() == bi


# ----------------------------------------------------------------------------- routing recipes
def test_softmax_routing_closed_form(oracle):
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(50, 8, generator=g)
    w, ids = oracle.route_softmax_topk(logits, 2)
    tv, ti = torch.topk(logits, 2, dim=-1)
    assert torch.equal(ids.long(), ti)
    # renormalised softmax over the picks == softmax over the picked logits alone
    assert torch.allclose(w, torch.softmax(tv, -1), rtol=1e-6, atol=1e-7)
    w_full, _ = oracle.route_softmax_topk(logits, 2, renorm=False)
    assert torch.allclose(w_full, torch.gather(torch.softmax(logits, -1), -1, ti))


def test_sigmoid_routing_matches_callers_recipe(oracle):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(32, 512, generator=g)
    wr = torch.randn(64, 512, generator=g) * 0.02        # keeps sigmoid away from saturation (no ties)
    want_w, want_ids = oracle.route_sigmoid_recipe(x, wr, 8)
    got_w, got_ids = oracle.route_sigmoid_grouped(x @ wr.T, None, 8, 1, 1, scale=2.5)
    assert torch.equal(got_ids.long(), want_ids)
    assert torch.allclose(got_w, want_w, rtol=1e-6)
    assert torch.allclose(got_w.sum(-1), torch.full((32,), 2.5))


def test_sigmoid_grouped_bias_only_moves_selection(oracle):
    g = torch.Generator().manual_seed(8)
    logits = torch.randn(16, 256, generator=g)
    bias = torch.zeros(256)
    bias[:32] = 10.0                                      # group 0 always wins, its experts too
    w, ids = oracle.route_sigmoid_grouped(logits, bias, 8, 8, 4)
    assert (ids < 32).all()
    s = torch.sigmoid(logits)
    picked = torch.gather(s, -1, ids.long())
    assert torch.allclose(w, picked / picked.sum(-1, keepdim=True) * 2.5)


# ----------------------------------------------------------------------------- permutation
@pytest.mark.parametrize("name", ["SELECTED_EXPERTS_B8_E256", "SELECTED_EXPERTS_B22_E256"])
def test_permutation_reference_tables(oracle, ref_fixtures, name):
    sel = torch.tensor(ref_fixtures[name], dtype=torch.int32)
    T, K = sel.shape
    assert K == 8 and all(len(set(r)) == K for r in sel.tolist())
    gather, scatter = oracle.permute_literal(sel, 256)
    sorted_slot, offsets, slot_to_row = oracle.permute_counting_sort(sel, 256)
    for e in range(256):
        seg = sorted_slot[offsets[e]:offsets[e + 1]].tolist()
        assert seg == scatter[e]
        assert [s // K for s in seg] == gather[e]
    assert offsets[-1].item() == T * K
    assert sorted(sorted_slot.tolist()) == list(range(T * K))
    assert torch.equal(slot_to_row[sorted_slot.long()], torch.arange(T * K, dtype=torch.int32))


def test_permutation_random_bruteforce_and_invariants(oracle):
    rng = random.Random(9)
    for T, E, K in [(1, 1, 1), (5, 4, 2), (37, 16, 4), (64, 8, 8), (3, 300, 5)]:
        sel = torch.tensor([rng.sample(range(E), K) for _ in range(T)], dtype=torch.int32)
        gather, scatter = oracle.permute_literal(sel, E)
        sorted_slot, offsets, _ = oracle.permute_counting_sort(sel, E)
        flat = sel.flatten()
        assert torch.equal(offsets[1:] - offsets[:-1], torch.bincount(flat.long(), minlength=E).int())
        keys = flat[sorted_slot.long()]
        assert (keys[1:] >= keys[:-1]).all()
        for e in range(E):
            assert sorted_slot[offsets[e]:offsets[e + 1]].tolist() == scatter[e]


def test_permutation_rejects_bad_ids(oracle):
    with pytest.raises(ValueError):
        oracle.permute_counting_sort(torch.tensor([[0, 9]], dtype=torch.int32), 8)


# ----------------------------------------------------------------------------- expert math
def _ref_layer(E, H, I, seed):
    g = torch.Generator().manual_seed(seed)
    w0 = (torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn)
    w1 = (torch.randn(E, I, H, generator=g) * 0.1).to(torch.float8_e4m3fn)
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(torch.float8_e4m3fn)
    s0 = (torch.randn(E, I // 128, H // 128, generator=g) * 0.1).to(torch.bfloat16)
    s1 = (torch.randn(E, I // 128, H // 128, generator=g) * 0.1).to(torch.bfloat16)
    s2 = (torch.randn(E, H // 128, I // 128, generator=g) * 0.1).to(torch.bfloat16)
    return w0, w1, w2, s0, s1, s2


def test_reference_form_literal_equals_vectorised(oracle):
    E, H, I, T, K = 4, 256, 128, 3, 2
    w = _ref_layer(E, H, I, 10)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    sel = torch.tensor([[0, 3], [2, 1], [3, 0]], dtype=torch.int32)
    a = oracle.experts_ref_bf16_literal(x, sel, *w)
    b = oracle.experts_ref_bf16(x, sel, *w)
    assert a.dtype == torch.bfloat16 and tuple(a.shape) == (T, K, H)
    # single rows vs batched rows can round the bf16 GEMM differently in the last place
    assert torch.allclose(a.float(), b.float(), rtol=2e-2, atol=1e-3)


def test_single_expert_reduces_to_dense_mlp(oracle):
    H, I = 256, 256
    w0, w1, w2, s0, s1, s2 = _ref_layer(1, H, I, 12)
    g = torch.Generator().manual_seed(13)
    x = torch.randn(5, H, generator=g).to(torch.bfloat16)
    sel = torch.zeros(5, 1, dtype=torch.int32)
    moe = oracle.experts_ref_bf16(x, sel, w0, w1, w2, s0, s1, s2)[:, 0]
    d0, d1, d2 = (oracle.dequant_block(w[0], s[0], 128, torch.bfloat16) for w, s in ((w0, s0), (w1, s1), (w2, s2)))
    dense = F.linear(F.silu(F.linear(x, d0)) * F.linear(x, d1), d2)
    assert torch.equal(moe, dense)


def test_w8a8_exact_when_quantisation_is_lossless(oracle):
    """With every 128-group hitting amax 448 and all values on the e4m3 grid, both
    activation and weight quantisation are exact, so the first GEMM + SwiGLU must equal a
    plain fp32 computation; the second GEMM then sees the (pinned) requantised h."""
    g = torch.Generator().manual_seed(14)
    grid = oracle.e4m3_decode_table()[[0x30, 0x34, 0x38, 0x3C, 0x40, 0xB0, 0xB8, 0xC0, 0x00]]
    E, H, I, T = 2, 256, 128, 4

    def on_grid(*shape):
        idx = torch.randint(0, len(grid), shape, generator=g)
        t = torch.from_numpy(grid)[idx].clone()
        return t

    x = on_grid(T, H)
    x[:, 0] = 448.0
    x[:, 128] = -448.0
    w13 = on_grid(E, 2 * I, H)
    w13[:, ::128, ::128] = 448.0
    w2 = on_grid(E, H, I)
    w2[:, ::128, ::128] = 448.0
    w13q, w13s = oracle.quant_weight_block128(w13)
    w2q, w2s = oracle.quant_weight_block128(w2)
    assert torch.equal(w13s, torch.ones_like(w13s)) and torch.equal(w13q.float(), w13)
    sel = torch.tensor([[0, 1], [1, 0], [0, 1], [1, 0]], dtype=torch.int32)
    out, (xq, xs, hq, hs) = oracle.experts_w8a8_fp32(x.to(torch.bfloat16), sel, w13q, w13s, w2q, w2s, return_mid=True)
    assert torch.equal(xq.float(), x) and torch.equal(xs, torch.ones_like(xs))
    for t in range(T):
        for k in range(2):
            e = int(sel[t, k])
            gu = F.linear(x[t], w13[e])
            h = F.silu(gu[:I]) * gu[I:]
            hq_ref, hs_ref = oracle.act_quant_group128(h[None])
            assert torch.equal(hq[t, k].view(torch.uint8), hq_ref[0].view(torch.uint8))
            assert torch.equal(hs[t, k], hs_ref[0])
            y = F.linear(oracle.act_dequant_group128(hq_ref, hs_ref)[0], w2[e])
            assert torch.allclose(out[t, k], y, rtol=1e-5, atol=1e-3 * y.abs().max().item())


def test_w8a8_close_to_unquantised_math(oracle):
    E, H, I, T, K = 4, 256, 256, 8, 2
    w13q, w13s, w2q, w2s = oracle.make_layer(E, H, I, seed=15)
    g = torch.Generator().manual_seed(16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    sel = torch.tensor([random.Random(t).sample(range(E), K) for t in range(T)], dtype=torch.int32)
    out = oracle.experts_w8a8_fp32(x, sel, w13q, w13s, w2q, w2s)
    w13 = oracle.dequant_block(w13q, w13s)
    w2 = oracle.dequant_block(w2q, w2s)
    for t in range(T):
        for k in range(K):
            e = int(sel[t, k])
            gu = F.linear(x[t].float(), w13[e])
            y = F.linear(F.silu(gu[:I]) * gu[I:], w2[e])
            assert oracle.cos_sim(y.numpy(), out[t, k].numpy()) > 0.995


def test_weighted_reduce_and_linearity(oracle):
    g = torch.Generator().manual_seed(17)
    y = torch.randn(5, 3, 16, generator=g)
    w = torch.rand(5, 3, generator=g)
    out = oracle.weighted_reduce(y, w)
    for t in range(5):
        acc = sum(w[t, k] * y[t, k] for k in range(3))
        assert torch.allclose(out[t], acc, rtol=1e-6, atol=1e-6)
    assert torch.allclose(oracle.weighted_reduce(y, 2 * w), 2 * out)


def test_moe_with_shared_expert_adds_dense_path(oracle):
    E, H, I, T, K = 4, 256, 128, 6, 2
    w13q, w13s, w2q, w2s = oracle.make_layer(E, H, I, seed=18)
    sh = oracle.make_layer(1, H, 256, seed=19)
    g = torch.Generator().manual_seed(20)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    sel = torch.tensor([[0, 1], [1, 2], [2, 3], [3, 0], [0, 2], [1, 3]], dtype=torch.int32)
    w = torch.rand(T, K, generator=g)
    base = oracle.moe_w8a8_fp32(x, sel, w, w13q, w13s, w2q, w2s)
    both = oracle.moe_w8a8_fp32(x, sel, w, w13q, w13s, w2q, w2s, shared=sh)
    dense = oracle.experts_w8a8_fp32(x, torch.zeros(T, 1, dtype=torch.int32), *sh)[:, 0]
    assert torch.allclose(both - base, dense, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- metrics
def test_metrics(oracle):
    a = np.array([1.0, 2.0, 3.0])
    assert oracle.cos_sim(a, a) == pytest.approx(1.0)
    assert oracle.cos_sim(a, -a) == pytest.approx(0.0)
    assert oracle.cos_sim(np.array([1.0, 0.0]), np.array([0.0, 1.0])) == pytest.approx(0.5)
    t = torch.tensor([3.0, 4.0])
    cd, rmse, amax = oracle.cal_diff(t, t)
    assert cd == pytest.approx(0.0) and rmse == 0 and amax == 0
    cd, rmse, amax = oracle.cal_diff(t, torch.tensor([3.0, 2.0]))
    assert amax == 2.0 and rmse == pytest.approx(math.sqrt(2.0)) and cd == pytest.approx(1 - 2 * 17 / 38)


# ----------------------------------------------------------------------------- dense layers
def test_dense_refs_reduce_to_library_routines(oracle):
    """scale == 1: the reference-form dense layers are plain F.linear chains on the cast weights;
    a ragged output width (576 = 4.5 blocks) uses the fifth scale row for its last 64 rows."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(5)
    M, K, N = 6, 256, 576
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    ones = torch.ones(5, 2, dtype=torch.bfloat16)
    assert torch.equal(oracle.mm_w8a16_dq_ref(x, w, ones), F.linear(x, w.to(torch.bfloat16)))
    s = ones.clone()
    s[4, :] = 2.0                                                  # only rows 512..575 are doubled
    y = oracle.mm_w8a16_dq_ref(x, w, s).float()
    y1 = F.linear(x, w.to(torch.bfloat16)).float()
    assert torch.equal(y[:, :512], y1[:, :512]) and torch.equal(y[:, 512:], 2 * y1[:, 512:])
    I = 128
    wg = torch.randn(I, K, generator=g).to(torch.float8_e4m3fn)
    wu = torch.randn(I, K, generator=g).to(torch.float8_e4m3fn)
    wd = torch.randn(K, I, generator=g).to(torch.float8_e4m3fn)
    one_a, one_b = torch.ones(1, 2, dtype=torch.bfloat16), torch.ones(2, 1, dtype=torch.bfloat16)
    want = F.linear(F.silu(F.linear(x, wg.to(torch.bfloat16))) * F.linear(x, wu.to(torch.bfloat16)), wd.to(torch.bfloat16))
    assert torch.equal(oracle.mlp_w8a16_dq_ref(x, wg, wu, wd, one_a, one_a, one_b), want)


def test_dense_w8a8_against_brute_force(oracle):
    """mm_w8a8_fp32 on a tiny case, element by element in python floats from the quantised operands;
    mlp_w8a8_fp32 == the single-expert MoE (already pinned) and its pieces chain through mm_w8a8_fp32."""
    g = torch.Generator().manual_seed(6)
    M, K, N = 3, 256, 16
    x = (torch.randn(M, K, generator=g) * 3).to(torch.bfloat16)
    wq, ws = oracle.quant_weight_block128(torch.randn(128, K, generator=g) * 0.05)
    wq, ws = wq[:N], ws                                            # ragged: 16 rows of one 128-row block
    got = oracle.mm_w8a8_fp32(x, wq, ws)
    xq, xs = oracle.act_quant_group128(x)
    tab = oracle.e4m3_decode_table()
    for m in range(M):
        for n in range(N):
            acc = 0.0
            for k in range(K):
                a = float(tab[int(xq.view(torch.uint8)[m, k])]) * float(xs[m, k // 128])
                b = float(tab[int(wq.view(torch.uint8)[n, k])]) * float(ws[0, k // 128])
                acc += a * b
            assert abs(acc - float(got[m, n])) <= 1e-5 * max(1.0, abs(acc))
    E, H, I = 1, 256, 128
    w13q, w13s, w2q, w2s = oracle.make_layer(E, H, I, seed=7)
    xx = torch.randn(5, H, generator=g).to(torch.bfloat16)
    y, (xq2, xs2, hq, hs) = oracle.mlp_w8a8_fp32(xx, w13q[0], w13s[0], w2q[0], w2s[0], return_mid=True)
    h = oracle.act_dequant_group128(hq[:, 0].view(torch.float8_e4m3fn), hs[:, 0])
    assert torch.allclose(y, h @ oracle.dequant_block(w2q[0], w2s[0]).T, rtol=1e-6, atol=1e-6)
