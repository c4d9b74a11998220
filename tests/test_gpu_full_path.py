"""The paths the benchmark times, at their real sizes, against the CPU oracle, through the C ABI on a real MI355X:

  * the DeepSeek-V3-shaped layer at T=4096 through the one-call entry point - router product on the matrix
    cores, 192-row tiles, the shared expert's tiles riding in the routed launches;
  * the same layer at decode sizes T = 1, 8, 32 (two-launch front end, 16/32-row tiles, narrow second GEMM).

The oracle cannot run a whole 11 GB layer; what is compared is (a) the router's logits for every token against an
fp64 product, (b) ids and weights for every token, exactly, given the scores the device selected on, (c) a sample
of tokens through the strict steps of oracle/parity_checks.py with only the experts they use brought to the host,
and (d) bit-equality of the big batch's rows with the staged kernels on the sampled tokens alone.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

H, I, E, K, I_SH = 7168, 2048, 256, 8, 2048
G, TG, SCALE = 8, 4, 2.5


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ds_layer(pkg, dev):
    """The DeepSeek-V3-shaped layer (256 routed experts + 1 shared), random weights made on the device."""
    say("building the full-size layer")
    layer = (*pkg.synthetic_weights(E, 2 * I, H, dev, 1), *pkg.synthetic_weights(E, H, I, dev, 2))
    shared = (*pkg.synthetic_weights(1, 2 * I_SH, H, dev, 3), *pkg.synthetic_weights(1, H, I_SH, dev, 4))
    g = torch.Generator(device=dev).manual_seed(5)
    wr = (torch.randn(E, H, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    yield layer, shared, wr
    del layer, shared, wr
    torch.cuda.empty_cache()


def _check_router(pkg, oracle, x, wr, bias, logits, w, ids):
    """(a) + (b) for every token of the batch."""
    exact = x.double().cpu() @ wr.double().cpu().t()
    err = (logits.double().cpu() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4 * x.double().cpu().norm(dim=1, keepdim=True) * wr.double().cpu().norm(dim=1)[None]
    assert bool((err <= bound).all()), float((err - bound).max())
    # the stand-alone routing entry point on the same logits: same bits, and it shows the scores it selected on
    w2, ids2, scores = pkg.moe_route(logits, K, "sigmoid", bias=bias, n_groups=G, topk_groups=TG, renorm=True,
                                     scale=SCALE, return_scores=True)
    assert torch.equal(ids, ids2) and torch.equal(w, w2)
    scores = scores.cpu()
    assert torch.allclose(scores, torch.sigmoid(logits.float().cpu()), rtol=1e-6, atol=1e-7)
    w_ref, ids_ref = oracle.select_sigmoid_grouped(scores, None if bias is None else bias.cpu(), K, G, TG, SCALE, True)
    assert torch.equal(ids.cpu(), ids_ref), "routing ids differ from the oracle's on the device's scores"
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    assert all(len(set(row)) == K for row in ids_ref.tolist())


def test_timed_prefill_path_deepseek_shape_with_shared_expert(pkg, oracle, dev, checks, ds_layer):
    layer, shared, wr = ds_layer
    T = 4096
    say("C3 timed path, T =", T, "tile rows", pkg.tile_rows(T, K, E))
    assert pkg.tile_rows(T, K, E) == 192
    g = torch.Generator(device=dev).manual_seed(11)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    bias = torch.zeros(E, device=dev)
    out, logits, w, ids = pkg.layer_fp8(x, wr, *layer, K, "sigmoid", bias=bias, n_groups=G, topk_groups=TG, renorm=True,
                                        scale=SCALE, shared=shared, return_routing=True)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    _check_router(pkg, oracle, x, wr, bias, logits, w, ids)
    # permutation of the whole batch
    ss, off, s2r = pkg.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids.cpu(), E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)
    # the staged entry point on the same routing gives the same bits as the one-call entry point
    out2 = pkg.fused_experts_fp8(x, *layer, ids, w, shared=shared)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    # sampled tokens: first and last of the batch, rows that land in different row tiles of their experts
    pick = torch.tensor([0, 1, 517, 1033, 2048, 2999, 3584, 4095], device=dev)
    y = pkg.fused_experts_fp8(x, *layer, ids)                    # per-slot rows of the whole batch, 192-row tiles
    torch.cuda.synchronize()
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), layer,
                              w_s=w[pick].contiguous(), shared_dev=shared, y_big=y[pick].contiguous(),
                              out_big=out[pick].contiguous(), what="C3 T=4096")
    say("   ", rep)


@pytest.mark.parametrize("T", [1, 8, 32])
def test_decode_deepseek_shape_full_size(pkg, oracle, dev, checks, ds_layer, T):
    layer, shared, wr = ds_layer
    say("C4 decode, T =", T, "tile rows", pkg.tile_rows(T, K, E))
    g = torch.Generator(device=dev).manual_seed(100 + T)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    bias = torch.zeros(E, device=dev)               # uniform router bias
    out, logits, w, ids = pkg.layer_fp8(x, wr, *layer, K, "sigmoid", bias=bias, n_groups=G, topk_groups=TG, renorm=True,
                                        scale=SCALE, shared=shared, return_routing=True)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    _check_router(pkg, oracle, x, wr, bias, logits, w, ids)
    ss, off, s2r = pkg.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids.cpu(), E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)
    # per-slot rows of the whole batch, then the sample against the oracle (the whole batch up to 8 tokens)
    y = pkg.fused_experts_fp8(x, *layer, ids)
    torch.cuda.synchronize()
    pick = torch.arange(T, device=dev) if T <= 8 else torch.tensor([0, 5, 13, 21, 30, 31], device=dev)
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), layer,
                              w_s=w[pick].contiguous(), shared_dev=shared, y_big=y[pick].contiguous(),
                              out_big=out[pick].contiguous(), what=f"C4 T={T}")
    say("   ", rep)
    # a second call gives the same bits
    again = pkg.layer_fp8(x, wr, *layer, K, "sigmoid", bias=bias, n_groups=G, topk_groups=TG, renorm=True, scale=SCALE,
                          shared=shared)
    torch.cuda.synchronize()
    assert torch.equal(again.view(torch.int16), out.view(torch.int16))


def _router_logits_close(x, wr, logits):
    exact = x.double().cpu() @ wr.double().cpu().t()
    err = (logits.double().cpu() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4 * x.double().cpu().norm(dim=1, keepdim=True) * wr.double().cpu().norm(dim=1)[None]
    assert bool((err <= bound).all()), float((err - bound).max())


def _timed_softmax_step(pkg, oracle, checks, dev, T, Hh, Ii, Ee, Kk, bias, pick, what, tile):
    """One call of the layer entry point as the benchmark times it (router product, softmax routing, permutation,
    quantisation, both grouped GEMMs, weighted sum) at the workload's full size: logits against an fp64 product,
    ids / weights exactly given the device's logits, permutation exactly, and sampled tokens of the batch's OWN
    output through the strict steps of oracle/parity_checks.py."""
    say(what, "timed path, T =", T, "tile rows", pkg.tile_rows(T, Kk, Ee))
    assert pkg.tile_rows(T, Kk, Ee) == tile
    layer = (*pkg.synthetic_weights(Ee, 2 * Ii, Hh, dev, 1), *pkg.synthetic_weights(Ee, Hh, Ii, dev, 2))
    g = torch.Generator(device=dev).manual_seed(5)
    wr = (torch.randn(Ee, Hh, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    gx = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, Hh, generator=gx, device=dev).to(torch.bfloat16)
    mode = "softmax" if bias is None else "softmax_logit_bias"
    out, logits, w, ids = pkg.layer_fp8(x, wr, *layer, Kk, mode, bias=bias, renorm=True, return_routing=True)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    _router_logits_close(x, wr, logits)
    lg = logits.float().cpu() if bias is None else logits.float().cpu() + bias.cpu()
    w_ref, ids_ref = oracle.route_softmax_topk(lg, Kk, True)
    assert torch.equal(ids.cpu(), ids_ref), "routing ids differ from the oracle's on the device's logits"
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ss, off, s2r = pkg.moe_permute(ids, Ee)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids_ref, Ee)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)
    # the staged entry point on the same routing: same bits
    out2 = pkg.fused_experts_fp8(x, *layer, ids, w)
    y = pkg.fused_experts_fp8(x, *layer, ids)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    pick = pick.to(dev)
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), layer,
                              w_s=w[pick].contiguous(), y_big=y[pick].contiguous(), out_big=out[pick].contiguous(),
                              what=what)
    say("   ", rep)
    return off_ref


def test_timed_prefill_path_mixtral_shape(pkg, oracle, dev, checks):
    """The Mixtral-8x7B-shaped step the benchmark reports under other_shapes (T=4096, E=8, top-2, 1024 rows per expert)."""
    _timed_softmax_step(pkg, oracle, checks, dev, 4096, 4096, 14336, 8, 2, None,
                        torch.tensor([0, 7, 1900, 3333, 4095]), "C2 T=4096", 192)
    torch.cuda.empty_cache()


def test_timed_prefill_path_skewed_load(pkg, oracle, dev, checks):
    """The Qwen3-30B-A3B-shaped step under the skewed load (T=16384, E=128, top-8; popularity ~ rank^-1.2 through a bias
    on the logits, 13 experts switched off): experts with thousands of rows next to experts with a handful and none."""
    Ee = 128
    g = torch.Generator(device=dev).manual_seed(5)
    torch.randn(Ee, 2048, generator=g, device=dev)              # the router weight's draw comes first, as in the benchmark
    rank = torch.randperm(Ee, generator=g, device=dev).float() + 1
    bias = -1.2 * torch.log(rank)
    dead = torch.randperm(Ee, generator=g, device=dev)[:13]
    bias[dead] = -1e9
    off = _timed_softmax_step(pkg, oracle, checks, dev, 16384, 2048, 768, Ee, 8, bias,
                              torch.tensor([0, 5000, 11111, 12345, 16383]), "C5 T=16384", 192)
    counts = off[1:] - off[:-1]
    assert int((counts[dead.cpu()] == 0).all()) and int((counts == 0).sum()) >= 13 and int(counts.max()) > 4000
    torch.cuda.empty_cache()
