"""Edge cases of the HIP path through the C ABI: empty batches, ids outside [0, E), a workspace that
is reused by calls of different sizes, and the largest expert / top-k counts."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def test_empty_batch_is_a_valid_call_everywhere(pkg, oracle, dev):
    say("empty batch")
    H, I, E, K = 256, 128, 8, 2
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=3)))
    x = torch.empty(0, H, dtype=torch.bfloat16, device=dev)
    ids = torch.empty(0, K, dtype=torch.int32, device=dev)
    w = torch.empty(0, K, dtype=torch.float32, device=dev)
    wr = torch.zeros(E, H, dtype=torch.bfloat16, device=dev)
    # routing
    wt, idx = pkg.moe_route(torch.empty(0, E, device=dev), K, "softmax")
    assert wt.shape == (0, K) and idx.shape == (0, K)
    v = torch.empty(0, K, device=dev)
    i = torch.empty(0, K, dtype=torch.int32, device=dev)
    pkg.noaux_tc_topk(v, i, torch.empty(0, E, device=dev), 1, 1, K)
    # permutation: nothing to place, every expert starts and ends at row 0
    ss, off, s2r = pkg.moe_permute(ids, E)
    torch.cuda.synchronize()
    assert ss.numel() == 0 and s2r.numel() == 0 and torch.equal(off.cpu(), torch.zeros(E + 1, dtype=torch.int32))
    # quantiser, experts (both output forms), un-quantised experts, dense layers, the one-call layer
    q, s = pkg.act_quant(x)
    assert q.shape == (0, H)
    assert pkg.fused_experts_fp8(x, *ld, ids).shape == (0, K, H)
    assert pkg.fused_experts_fp8(x, *ld, ids, w).shape == (0, H)
    w13b = torch.zeros(E, 2 * I, H, dtype=torch.bfloat16, device=dev)
    w2b = torch.zeros(E, H, I, dtype=torch.bfloat16, device=dev)
    assert pkg.fused_experts_bf16(x, w13b, w2b, ids, w).shape == (0, H)
    assert pkg.fused_experts_w8a16(x, *ld, ids).shape == (0, K, H)
    assert pkg.fused_experts_w8a16(x, *ld, ids, w).shape == (0, H)
    assert pkg.mm_w8a16(x, ld[0][0], ld[1][0]).shape == (0, 2 * I)
    assert pkg.mm_fp8(x, ld[0][0], ld[1][0]).shape == (0, 2 * I)
    assert pkg.mlp_fp8(x, ld[0][0], ld[1][0], ld[2][0], ld[3][0]).shape == (0, H)
    moe = pkg.FusedMoE(wr, *ld, top_k=K, mode="softmax")
    assert moe(x).shape == (0, H)
    torch.cuda.synchronize()


def test_ids_outside_the_expert_range_are_dropped(pkg, oracle, dev):
    say("ids out of range")
    T, E, K = 37, 16, 4
    g = torch.Generator().manual_seed(9)
    ids = torch.argsort(torch.rand(T, E, generator=g), dim=-1)[:, :K].to(torch.int32)
    bad = torch.rand(T, K, generator=g) < 0.2
    ids[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, torch.tensor(-1), torch.tensor(E + 3)).to(torch.int32)
    ss, off, s2r = pkg.moe_permute(ids.to(dev), E)
    torch.cuda.synchronize()
    flat = ids.flatten()
    valid = (flat >= 0) & (flat < E)
    n_valid = int(valid.sum())
    counts = torch.bincount(flat[valid].long(), minlength=E)
    off_ref = torch.zeros(E + 1, dtype=torch.int64)
    off_ref[1:] = torch.cumsum(counts, 0)
    assert torch.equal(off.cpu().long(), off_ref)
    # the valid slots in stable expert order, the dropped ones nowhere
    order = torch.sort(torch.where(valid, flat, torch.tensor(E, dtype=torch.int32)).long(), stable=True).indices[:n_valid]
    assert torch.equal(ss.cpu()[:n_valid].long(), order)
    s2r = s2r.cpu()
    assert bool((s2r[~valid] == -1).all())
    inv = torch.full((T * K,), -1, dtype=torch.int64)
    inv[order] = torch.arange(n_valid)
    assert torch.equal(s2r.long(), inv)


@pytest.mark.parametrize("T", [5, 37, 300])
def test_slots_without_an_expert_add_nothing(pkg, oracle, dev, T):
    """Ids outside [0, E) (how an expert-parallel rank marks the experts it does not hold): zero rows in the
    [T, K, H] form, no term in the weighted sum, everything else as if the slot were not there."""
    say("dropped slots in the expert computation", T)
    H, I, E, K = 256, 128, 8, 3
    layer = oracle.make_layer(E, H, I, seed=12)
    g = torch.Generator().manual_seed(12 + T)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.argsort(torch.rand(T, E, generator=g), dim=-1)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    bad = torch.rand(T, K, generator=g) < 0.3
    bad[0] = True                                            # a token none of whose slots has an expert
    ids_bad = ids.clone()
    ids_bad[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, torch.tensor(-1), torch.tensor(E)).to(torch.int32)
    ref_slots = oracle.experts_w8a8_fp32(x, ids, *layer)
    ref_slots[bad] = 0.0
    dl = pkg.pack_layer(*(t.to(dev) for t in layer))
    # poisoned outputs and workspace: whatever the call does not write would show
    out3 = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.fused_experts_fp8(x.to(dev), *dl, ids_bad.to(dev), out=out3)
    torch.cuda.synchronize()
    got3 = out3.float().cpu()
    assert torch.isfinite(got3).all()
    assert bool((got3[bad] == 0).all())
    scale = ref_slots.abs().max().item()
    frac = ((got3 - ref_slots).abs() > (1e-2 + 2e-2 * ref_slots.abs() / scale) * scale).float().mean().item()
    assert frac <= 5e-3
    ws = torch.empty(pkg.fused_experts_workspace_bytes(T, H, I, E, K), dtype=torch.uint8, device=dev)
    ws.view(torch.int16)[: ws.numel() // 2].fill_(0x7FC0)       # bf16 NaN everywhere
    out2 = pkg.fused_experts_fp8(x.to(dev), *dl, ids_bad.to(dev), w.to(dev), workspace=ws)
    torch.cuda.synchronize()
    got2 = out2.float().cpu()
    assert torch.isfinite(got2).all()
    assert bool((got2[0] == 0).all())
    ref2 = torch.einsum("tk,tkh->th", w, got3)                  # the device's own slot results, summed on the host
    torch.testing.assert_close(got2, ref2, rtol=2e-2, atol=1e-2 * scale)
    # un-quantised experts take the same route
    w13b = pkg.pack_weights(oracle.dequant_block(layer[0], layer[1]).to(torch.bfloat16).to(dev))
    w2b = pkg.pack_weights(oracle.dequant_block(layer[2], layer[3]).to(torch.bfloat16).to(dev))
    outb = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.fused_experts_bf16(x.to(dev), w13b, w2b, ids_bad.to(dev), out=outb)
    torch.cuda.synchronize()
    assert torch.isfinite(outb.float()).all() and bool((outb.float().cpu()[bad] == 0).all())
    outb2 = pkg.fused_experts_bf16(x.to(dev), w13b, w2b, ids_bad.to(dev), w.to(dev))
    torch.cuda.synchronize()
    assert torch.isfinite(outb2.float()).all() and bool((outb2.float().cpu()[0] == 0).all())
    # and so does the reference's arithmetic on the packed FP8 weights
    outd = torch.full((T, K, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.fused_experts_w8a16(x.to(dev), *dl, ids_bad.to(dev), out=outd)
    outd2 = pkg.fused_experts_w8a16(x.to(dev), *dl, ids_bad.to(dev), w.to(dev))
    torch.cuda.synchronize()
    gotd = outd.float().cpu()
    assert torch.isfinite(gotd).all() and bool((gotd[bad] == 0).all())
    assert torch.isfinite(outd2.float()).all() and bool((outd2.float().cpu()[0] == 0).all())
    live = ~bad
    assert oracle.cal_diff(ref_slots[live], gotd[live])[0] < 5e-3      # un-quantised activations against the W8A8 oracle


def test_one_workspace_serves_calls_of_different_sizes(pkg, oracle, dev):
    say("workspace reuse")
    H, I, E, K = 512, 256, 16, 4
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=4)))
    sizes = [300, 3, 70, 1, 129]
    ws = torch.empty(pkg.fused_experts_workspace_bytes(max(sizes), H, I, E, K), dtype=torch.uint8, device=dev)
    ws.fill_(0xA5)
    g = torch.Generator().manual_seed(4)
    for T in sizes:
        x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
        ids = torch.argsort(torch.rand(T, E, generator=g), dim=-1)[:, :K].to(torch.int32).to(dev)
        w = torch.rand(T, K, generator=g).to(dev)
        shared_ws = pkg.fused_experts_fp8(x, *ld, ids, w, workspace=ws)
        fresh_ws = pkg.fused_experts_fp8(x, *ld, ids, w)
        assert torch.equal(shared_ws.view(torch.int16), fresh_ws.view(torch.int16)), T


def test_largest_expert_and_topk_counts(pkg, oracle, dev):
    say("E=1024, K=32")
    T, H, I, E, K = 40, 256, 128, 1024, 32
    layer = oracle.make_layer(E, H, I, seed=6)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    w_ref, ids_ref = oracle.route_softmax_topk(logits, K)
    w, ids = pkg.moe_route(logits.to(dev), K, "softmax")
    assert torch.equal(ids.cpu(), ids_ref)
    out = pkg.fused_experts_fp8(x.to(dev), *pkg.pack_layer(*(t.to(dev) for t in layer)), ids, w)
    torch.cuda.synchronize()
    ref = oracle.moe_w8a8_fp32(x, ids_ref, w_ref, *layer)
    bad = (out.float().cpu() - ref).abs() > 1e-2 + 2e-2 * ref.abs()
    assert bad.float().mean().item() <= 5e-3


def test_large_batch_addresses(pkg, oracle, dev):
    """A batch whose per-slot output is larger than 4 GB (and whose quantised intermediate is close to 1 GB): row
    addresses must be formed in 64 bits.  Tokens from both ends of the batch equal the same tokens run on their own."""
    say("large batch")
    T, H, I, E, K = 150000, 2048, 768, 32, 8
    gg = torch.Generator(device=dev).manual_seed(77)
    w13 = (torch.randn(E, 2 * I, H, generator=gg, device=dev) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, generator=gg, device=dev) * 0.02).to(torch.bfloat16)
    w13q, w13s = pkg.quant_weight_block128(w13)
    w2q, w2s = pkg.quant_weight_block128(w2)
    w13q, w2q = pkg.pack_weights(w13q), pkg.pack_weights(w2q)
    del w13, w2
    x = torch.randn(T, H, generator=gg, device=dev).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=gg, device=dev)
    w, ids = pkg.moe_route(logits, K, "softmax")
    assert T * K * H * 2 > (1 << 32) and T * K * I > (1 << 29)
    y = pkg.fused_experts_fp8(x, w13q, w13s, w2q, w2s, ids)
    out = pkg.fused_experts_fp8(x, w13q, w13s, w2q, w2s, ids, w)
    torch.cuda.synchronize()
    pick = torch.cat([torch.arange(0, 40), torch.arange(T // 2, T // 2 + 40), torch.arange(T - 40, T)]).to(dev)
    y_s = pkg.fused_experts_fp8(x[pick].contiguous(), w13q, w13s, w2q, w2s, ids[pick].contiguous())
    out_s = pkg.fused_experts_fp8(x[pick].contiguous(), w13q, w13s, w2q, w2s, ids[pick].contiguous(), w[pick].contiguous())
    torch.cuda.synchronize()
    assert torch.isfinite(y_s.float()).all() and float(y_s.float().abs().max()) > 0
    assert torch.equal(y[pick].view(torch.int16), y_s.view(torch.int16))
    assert torch.equal(out[pick].view(torch.int16), out_s.view(torch.int16))


def test_read_probe_reads_any_size_and_rejects_bad_arguments(pkg, dev):
    """bench.py's yardstick (bench_hbm_read_probe, a library of its own beside the product's): runs on sizes that its
    piece size does not divide, leaves the buffer alone, and refuses sizes that are not multiples of 16 bytes."""
    import bench
    buf = torch.arange(3 * 1000 * 16 + 16, dtype=torch.uint8, device=dev)
    before = buf.clone()
    for piece in (16, 4096, 1 << 20, 1 << 30):
        bench.hbm_read_probe(buf, piece)
    torch.cuda.synchronize()
    assert torch.equal(buf, before)
    with pytest.raises(RuntimeError):
        bench.hbm_read_probe(buf[:24])
    with pytest.raises(RuntimeError):
        bench.hbm_read_probe(buf, 24)


@pytest.mark.parametrize("counts", [[1, 97, 193, 1209], [96, 192, 288, 1000], [95, 191, 2, 1400], [0, 383, 385, 900]])
def test_half_tiles_at_the_edges_of_their_tiles(pkg, oracle, dev, checks, counts):
    """Experts with many rows and a short reduction run the 96-row half tiles on a 192-row tile list: expert row counts
    that end exactly at, one before and one after the halves' and the list tiles' edges (and an expert without a row),
    every token against the oracle through the strict steps, and the batch's rows equal to the same tokens run alone."""
    say("half tiles, rows per expert", counts)
    E, K, H, I = len(counts), 1, 256, 256
    T = sum(counts)
    assert T * K / E >= 320 and H // 128 <= 20 and pkg.tile_rows(T, K, E) == 192      # the launcher's rule for half tiles
    ids = torch.cat([torch.full((n,), e, dtype=torch.int32) for e, n in enumerate(counts)])
    g = torch.Generator().manual_seed(sum(counts))
    ids = ids[torch.randperm(T, generator=g)].reshape(T, 1).contiguous()
    w = torch.rand(T, 1, generator=g) + 0.5
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=7)))
    xd, idd, wd = x.to(dev), ids.to(dev), w.to(dev)
    y = pkg.fused_experts_fp8(xd, *ld, idd)
    out = pkg.fused_experts_fp8(xd, *ld, idd, wd)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    # first and last rows of every expert (in permuted order those sit at the tiles' edges)
    order = torch.argsort(ids[:, 0], stable=True)
    edges = []
    pos = 0
    for n in counts:
        for r in (0, 95, 96, 97, 191, 192, 193, n - 1):
            if 0 <= r < n:
                edges.append(int(order[pos + r]))
        pos += n
    pick = torch.tensor(sorted(set(edges)), device=dev)
    rep = checks.check_sample(pkg, oracle, xd[pick].contiguous(), idd[pick].contiguous(), ld, w_s=wd[pick].contiguous(),
                              y_big=y[pick].contiguous(), out_big=out[pick].contiguous(), what="half tiles")
    say("   ", rep)
