"""The one-call layer entry point (moe_layer_fp8: router and experts) at decode sizes and beyond, and the
workgroup-per-token routing kernel, through the C ABI, on a real MI355X.

What must hold, bit for bit: the routing of a small batch equals the routing of the same rows inside
a large batch (two different kernels) and the oracle's ids; given the logits the entry point produced, its
ids and weights equal moe_route_topk's; given those, its output equals moe_fused_experts_fp8's.
The logits themselves are a bf16 rounding of an fp32 dot product: checked against an fp64 product with
the tolerance of that rounding.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


ROUTE_CASES = [
    # E, K, mode, groups, kept groups, bias, ties
    (8, 2, "softmax", 1, 1, False, False),
    (128, 8, "softmax", 1, 1, False, True),
    (200, 6, "softmax", 1, 1, True, False),
    (256, 8, "sigmoid", 8, 4, True, False),
    (256, 8, "sigmoid", 8, 4, False, True),
    (96, 7, "sigmoid", 3, 2, True, True),
    (64, 32, "scores", 4, 3, False, True),
    (250, 5, "sigmoid", 1, 1, False, False),
]


@pytest.mark.parametrize("E,K,mode,G,TG,with_bias,ties", ROUTE_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_batch_routing_equals_large_batch_routing(pkg, oracle, dev, E, K, mode, G, TG, with_bias, ties, dtype):
    say("route small vs large", E, K, mode, G, TG, with_bias, ties, dtype)
    T = 150                                            # above the small-batch limit: one wavefront per token
    g = torch.Generator().manual_seed(E * 31 + K)
    logits = torch.randn(T, E, generator=g) * 1.5
    if mode == "scores":
        logits = torch.rand(T, E, generator=g)
    if ties:
        logits[::2] = torch.round(logits[::2] * 2) / 2  # many exact ties, in the groups' sums as well
        logits[3] = 0.25                                # one row of a single value
    logits = logits.to(dtype).to(dev)
    bias = (torch.randn(E, generator=g) * 0.1).to(dev) if with_bias else None
    kw = dict(bias=bias, n_groups=G, topk_groups=TG, renorm=True, scale=2.5, return_scores=True)
    w_big, i_big, s_big = pkg.moe_route(logits, K, mode, **kw)
    for lo, n in ((0, 1), (1, 7), (8, 64), (100, 50)):
        w, i, s = pkg.moe_route(logits[lo:lo + n].contiguous(), K, mode, **kw)
        assert torch.equal(i, i_big[lo:lo + n]), (lo, n)
        assert torch.equal(w, w_big[lo:lo + n]), (lo, n)
        assert torch.equal(s, s_big[lo:lo + n]), (lo, n)
    w_nr, i_nr = pkg.moe_route(logits[:9].contiguous(), K, mode, bias=bias, n_groups=G, topk_groups=TG, renorm=False)
    w_nr_big, i_nr_big = pkg.moe_route(logits, K, mode, bias=bias, n_groups=G, topk_groups=TG, renorm=False)
    assert torch.equal(i_nr, i_nr_big[:9]) and torch.equal(w_nr, w_nr_big[:9])
    # and the ids are the oracle's, given the scores the device selected on
    small = pkg.moe_route(logits[:40].contiguous(), K, mode, **kw)
    scores = small[2].cpu()
    b = None if bias is None else bias.cpu()
    if mode == "softmax":
        # selection looks at the logits (+ bias); a softmax is monotone, so any row-wise top-k of them will do
        sel = logits[:40].float().cpu() + (0 if b is None else b)
        order = torch.sort(sel, dim=-1, descending=True, stable=True).indices[:, :K].to(torch.int32)
        assert torch.equal(small[1].cpu(), order)
    else:
        w_ref, i_ref = oracle.select_sigmoid_grouped(scores, b, K, G, TG, 2.5, True)
        assert torch.equal(small[1].cpu(), i_ref)
        assert torch.allclose(small[0].cpu(), w_ref, rtol=1e-5, atol=1e-7)


def _shared(pkg, oracle, H, I_sh, seed, dev):
    w13, w13s, w2, w2s = oracle.make_layer(1, H, I_sh, seed=seed)
    return pkg.pack_layer(*(t.to(dev) for t in (w13, w13s, w2, w2s)))


LAYER_CASES = [
    # T, H, I, E, K, mode, groups, kept, bias, shared I
    (1, 7168, 256, 256, 8, "sigmoid", 8, 4, True, 256),
    (8, 1024, 256, 64, 6, "softmax", 1, 1, False, 0),
    (32, 512, 384, 8, 2, "softmax", 1, 1, False, 0),
    (19, 1280, 128, 100, 4, "sigmoid", 4, 2, True, 384),
    (32, 2304, 128, 256, 8, "sigmoid", 8, 4, False, 128),
    (3, 8192 + 1024, 128, 16, 3, "sigmoid", 1, 1, False, 0),
    (8, 7168, 2048, 256, 8, "sigmoid", 8, 4, True, 2048),        # the DeepSeek-V3 layer at its real size
    # beyond the decode size: the router product on the matrix cores, reduction in slices
    (300, 1024, 256, 64, 6, "softmax", 1, 1, False, 0),
    (77, 512, 128, 8, 4, "sigmoid", 1, 1, True, 128),
    (1000, 7168, 256, 256, 8, "sigmoid", 8, 4, True, 256),
    (4096, 2048, 128, 250, 5, "sigmoid", 1, 1, False, 0),
]


@pytest.mark.parametrize("T,H,I,E,K,mode,G,TG,with_bias,I_sh", LAYER_CASES)
def test_layer_entry_point(pkg, oracle, dev, checks, T, H, I, E, K, mode, G, TG, with_bias, I_sh):
    run_layer_case(pkg, oracle, dev, checks, T, H, I, E, K, mode, G, TG, with_bias, I_sh)


def random_layer_case(seed):
    """Layer shape, batch size and router drawn from the seed: batches either side of the decode size, grouped sigmoid
    routing with at least two experts per group, or softmax."""
    import random
    r = random.Random(seed)
    mode = r.choice(["softmax", "sigmoid", "sigmoid"])
    G = r.choice([1, 1, 2, 4, 8]) if mode == "sigmoid" else 1
    per = r.choice([2, 3, 4, 8, 16, 32])
    E = min(256, G * per) if G > 1 else r.choice([2, 5, 8, 17, 64, 100, 256])
    per = E // G
    TG = r.randint(1, G)
    K = r.randint(1, min(8, TG * per))
    H, I = 128 * r.randint(1, 16), 128 * r.randint(1, 4)
    T = r.choice([1, 2, 3, 9, 16, 31, 32, 33, 64, 65, 129, 300, 700])
    I_sh = r.choice([0, I, 128 * r.randint(1, 3)])
    with_bias = r.random() < 0.5 and mode == "sigmoid"     # a softmax router's bias has a test of its own below
    return T, H, I, E, K, mode, G, TG, with_bias, I_sh


@pytest.mark.parametrize("seed", range(24))
def test_layer_entry_point_random_cases(pkg, oracle, dev, checks, seed):
    run_layer_case(pkg, oracle, dev, checks, *random_layer_case(500 + seed))


def run_layer_case(pkg, oracle, dev, checks, T, H, I, E, K, mode, G, TG, with_bias, I_sh):
    say("decode layer", T, H, I, E, K, mode, G, TG, with_bias, I_sh)
    small = 3 * E * H * I <= (1 << 26)
    if small:
        layer = oracle.make_layer(E, H, I, seed=T + E)
        ld = pkg.pack_layer(*(t.to(dev) for t in layer))
    else:                                   # too large to make on the host: random weights made on the device
        ld = (*pkg.synthetic_weights(E, 2 * I, H, dev, T + E), *pkg.synthetic_weights(E, H, I, dev, T + E + 1))
    g = torch.Generator().manual_seed(7 * T + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16)
    bias = (torch.randn(E, generator=g) * 0.05) if with_bias else None
    xd, wrd = x.to(dev), wr.to(dev)
    biasd = None if bias is None else bias.to(dev)
    shared = _shared(pkg, oracle, H, I_sh, 99, dev) if I_sh else None
    kw = dict(bias=biasd, n_groups=G, topk_groups=TG, renorm=True, scale=2.5 if mode == "sigmoid" else 1.0)

    out, logits, w, ids = pkg.layer_fp8(xd, wrd, *ld, K, mode, shared=shared, return_routing=True, **kw)
    torch.cuda.synchronize()
    # logits: bf16 rounding of the exact product
    exact = x.double() @ wr.double().t()
    err = (logits.double().cpu() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4 * x.double().norm(dim=1, keepdim=True) * wr.double().norm(dim=1)[None]
    assert bool((err <= bound).all()), float((err - bound).max())
    # routing: the stand-alone routing entry point on the same logits
    w2_, ids2 = pkg.moe_route(logits, K, mode, **kw)
    assert torch.equal(ids, ids2) and torch.equal(w, w2_)
    # experts: the stand-alone expert entry point on the same routing
    ref_out = pkg.fused_experts_fp8(xd, *ld, ids, w, shared=shared)
    assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16))
    # a second call into the same workspace (the arrival counter starts over), without the optional outputs
    ws = torch.empty(pkg.layer_workspace_bytes(T, H, I, E, K, I_sh), dtype=torch.uint8, device=dev)
    for _ in range(2):
        again = pkg.layer_fp8(xd, wrd, *ld, K, mode, shared=shared, workspace=ws, **kw)
        assert torch.equal(again.view(torch.int16), out.view(torch.int16))
    # the module takes this road by itself for such a batch
    moe = pkg.FusedMoE(wrd, *ld, top_k=K, mode=mode, bias=biasd, n_groups=G, topk_groups=TG, renorm=True,
                       scale=kw["scale"], shared=shared)
    assert moe._one_call(T)
    assert torch.equal(moe(xd).view(torch.int16), out.view(torch.int16))
    # and the whole thing against the oracle.  Routing is compared on the scores the device selected on (its
    # sigmoid may differ from the host's in the last place; the selection given the scores may not), so the
    # comparison always runs; the experts go through the strict steps on a sample of tokens.
    if mode == "softmax":
        w_ref, ids_ref = oracle.route_softmax_topk(logits.float().cpu(), K)
    else:
        scores = pkg.moe_route(logits, K, mode, return_scores=True, **kw)[2].cpu()
        assert torch.allclose(scores, torch.sigmoid(logits.float().cpu()), rtol=1e-6, atol=1e-7)
        w_ref, ids_ref = oracle.select_sigmoid_grouped(scores, bias, K, G, TG, 2.5, True)
    assert torch.equal(ids.cpu(), ids_ref), "routing ids differ from the oracle's on the device's scores"
    assert torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    pick = torch.arange(T) if T <= 12 else torch.unique(torch.linspace(0, T - 1, 10).long())
    pick = pick.to(dev)
    rep = checks.check_sample(pkg, oracle, xd[pick].contiguous(), ids[pick].contiguous(), ld, w_s=w[pick].contiguous(),
                              shared_dev=shared, out_big=out[pick].contiguous(), what=f"layer T={T} E={E}")
    say("   ", {k: (round(v, 6) if isinstance(v, float) else v) for k, v in rep.items()})


@pytest.mark.parametrize("T", [1, 5, 32, 300, 2000])
def test_softmax_router_whose_bias_is_part_of_the_logits(pkg, oracle, dev, T):
    """MOE_ROUTE_SOFTMAX_LOGIT_BIAS: softmax over logits + bias (selection and weights see the bias), the form a
    softmax router's own bias term takes - a skewed-load layer switches experts off with it.  One call through the
    layer entry point equals the staged road (logits + bias on the host side, plain softmax routing) bit for bit."""
    say("softmax router with a logit bias", T)
    H, I, E, K = 1024, 256, 64, 6
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=T + 1)))
    g = torch.Generator().manual_seed(17 * T + 3)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bias = -1.2 * torch.log(torch.randperm(E, generator=g).float() + 1)
    off = torch.randperm(E, generator=g)[:7]
    bias[off] = -1e9                                                   # experts that must never be chosen
    biasd = bias.to(dev)
    out, logits, w, ids = pkg.layer_fp8(x, wr, *ld, K, "softmax_logit_bias", bias=biasd, return_routing=True)
    w1, ids1 = pkg.moe_route(logits, K, "softmax_logit_bias", bias=biasd)
    w2_, ids2 = pkg.moe_route(logits.float() + biasd, K, "softmax")
    torch.cuda.synchronize()
    assert torch.equal(ids, ids1) and torch.equal(w, w1)
    assert torch.equal(ids, ids2) and torch.equal(w, w2_)
    assert not bool(torch.isin(ids.cpu().long(), off).any())
    w_ref, ids_ref = oracle.route_softmax_topk(logits.float().cpu() + bias, K)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ref_out = pkg.fused_experts_fp8(x, *ld, ids, w)
    assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16))
    # the module hands a softmax router's bias over in this form by itself
    moe = pkg.FusedMoE(wr, *ld, top_k=K, mode="softmax", bias=biasd)
    assert moe._one_call(T) and moe.layer_mode() == "softmax_logit_bias"
    assert torch.equal(moe(x).view(torch.int16), out.view(torch.int16))
    wm, im = moe.route(x)                                              # its staged road: the router product and the selection, call by call
    assert not bool(torch.isin(im.cpu().long(), off).any())


@pytest.mark.parametrize("T,H,E", [(1, 128, 1), (5, 7168, 256), (64, 256, 16), (65, 384, 100), (700, 7168, 256),
                                   (4096, 2048, 128), (130, 9216, 37), (3, 512, 257), (200, 1024, 384), (70, 256, 1024),
                                   (300, 384, 1000)])
def test_router_logits_kernel(pkg, dev, T, H, E):
    say("router logits", T, H, E)
    g = torch.Generator().manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16)
    got = pkg.router_logits(x.to(dev), wr.to(dev))
    again = pkg.router_logits(x.to(dev), wr.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), again.view(torch.int16))           # fixed summation order
    exact = x.double() @ wr.double().t()
    err = (got.double().cpu() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4 * x.double().norm(dim=1, keepdim=True) * wr.double().norm(dim=1)[None]
    assert bool((err <= bound).all()), float((err - bound).max())


def test_layer_entry_point_in_a_hip_graph(pkg, oracle, dev):
    say("decode layer graph")
    T, H, I, E, K = 4, 1024, 256, 64, 4
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=5)))
    g = torch.Generator().manual_seed(5)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    xs = [torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev) for _ in range(3)]
    moe = pkg.FusedMoE(wr, *ld, top_k=K, mode="softmax")
    eager = [moe(x).clone() for x in xs]
    x_static = xs[0].clone()
    out_static = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        moe(x_static, out=out_static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        moe(x_static, out=out_static)
    for rep in range(2):
        for x, ref in zip(xs, eager):
            x_static.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_static.view(torch.int16), ref.view(torch.int16)), rep
            assert torch.equal(moe(x).view(torch.int16), ref.view(torch.int16))     # eager work between replays


def test_shared_expert_beside_the_front_end_changes_no_bit(pkg, oracle, dev):
    """Batches of 512 tokens and more: the shared expert's first GEMM runs on a stream of the library's own beside the
    router product, routing and permutation.  Same bits as with that switched off, on the default stream and on a
    stream of the caller's, call after call into one workspace, and inside a graph capture (where the side stream is
    not used)."""
    say("shared expert beside the front end")
    T, H, I, E, K = 777, 1024, 256, 32, 4
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=11)))
    shared = _shared(pkg, oracle, H, I, 12, dev)
    g = torch.Generator().manual_seed(11)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    xs = [torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev) for _ in range(3)]
    kw = dict(shared=shared, n_groups=4, topk_groups=2, renorm=True, scale=2.5)
    was = pkg.set_shared_overlap(False)
    try:
        assert was is True
        plain = [pkg.layer_fp8(x, wr, *ld, K, "sigmoid", **kw).clone() for x in xs]
        assert pkg.set_shared_overlap(True) is False
        ws = torch.empty(pkg.layer_workspace_bytes(T, H, I, E, K, I), dtype=torch.uint8, device=dev)
        for rep in range(3):
            for x, ref in zip(xs, plain):
                got = pkg.layer_fp8(x, wr, *ld, K, "sigmoid", workspace=ws, **kw)
                assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), rep
        torch.cuda.synchronize()
        own = torch.cuda.Stream()
        own.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(own):
            ws2 = torch.empty_like(ws)
            got = [pkg.layer_fp8(x, wr, *ld, K, "sigmoid", workspace=ws2, **kw) for x in xs]
        torch.cuda.current_stream().wait_stream(own)
        for a, ref in zip(got, plain):
            assert torch.equal(a.view(torch.int16), ref.view(torch.int16))
        # under capture the call stays on the captured stream
        x_static, out_static = xs[0].clone(), torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            pkg.layer_fp8(x_static, wr, *ld, K, "sigmoid", out=out_static, workspace=ws, **kw)
        for rep in range(2):
            for x, ref in zip(xs, plain):
                x_static.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(out_static.view(torch.int16), ref.view(torch.int16)), rep
                assert torch.equal(pkg.layer_fp8(x, wr, *ld, K, "sigmoid", **kw).view(torch.int16), ref.view(torch.int16))
    finally:
        pkg.set_shared_overlap(True)


def test_layer_entry_point_rejects_what_it_does_not_cover(pkg, oracle, dev):
    say("layer entry errors")
    H, I = 256, 128
    g = torch.Generator().manual_seed(1)
    assert pkg.layer_eligible(33, 16, 8) and pkg.layer_eligible(4096, 256, 8)
    assert pkg.layer_eligible(1, 1024, 8) and not pkg.layer_eligible(1, 1025, 8) and not pkg.layer_eligible(1, 4, 8)
    lib = pkg._lib.lib
    # more than 1024 experts: refused on the shape alone, before anything is launched (the pointers are never used)
    assert lib.moe_layer_fp8(None, 1, 1, H, 1, None, 1300, 8, 0, 1, 1, 1, 1.0, 1, 1, 1, 1, I, None, None, None, None,
                             0, 1, None, None, None, 256, 1 << 30) == -2
    assert lib.moe_layer_fp8_workspace_bytes(1, H, I, 1300, 8, 0) == 0
    E, K = 16, 8
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=1)))
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    x = torch.randn(2, H, generator=g).to(torch.bfloat16).to(dev)
    with pytest.raises(RuntimeError):
        pkg.layer_fp8(x, wr, *ld, K, "scores")                       # not a routing mode of this entry point
    with pytest.raises(RuntimeError):
        pkg.layer_fp8(x, wr, *ld, K, "softmax", workspace=torch.empty(256, dtype=torch.uint8, device=dev))
    out = pkg.layer_fp8(x, wr, *ld, K, "softmax")
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()


def test_checkpoint_converter_feeds_the_kernels(pkg, oracle, dev, checks):
    """A DeepSeek-V3-style FP8 checkpoint (per-expert `weight` [out, in] + `weight_scale_inv`, router, correction bias,
    shared expert) through convert_hf_moe_layer into the module, against the oracle on the checkpoint's own tensors;
    and the reference's argument layout (separate gate / up, pre-transposed down and scales,
    python/regression/test_llm/test_moe.py:285-288) through pack_expert_weights gives the same packed bytes."""
    say("checkpoint converter")
    E, H, I, K, T = 16, 512, 256, 4, 24
    g = torch.Generator().manual_seed(31)
    state, pre = {}, "model.layers.3.mlp."
    per_expert = {}
    for e in list(range(E)) + ["s"]:
        base = pre + ("shared_experts." if e == "s" else f"experts.{e}.")
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            q, sc = oracle.quant_weight_block128(torch.randn(n, k, generator=g) * 0.05)
            state[base + proj + ".weight"], state[base + proj + ".weight_scale_inv"] = q, sc
            per_expert[(e, proj)] = (q, sc)
    state[pre + "gate.weight"] = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16)
    state[pre + "gate.e_score_correction_bias"] = torch.randn(E, generator=g) * 0.05
    conv = pkg.convert_hf_moe_layer(state, pre, E, device=dev)
    moe = pkg.FusedMoE(conv["router_weight"], conv["w13"], conv["w13_scale"], conv["w2"], conv["w2_scale"], top_k=K,
                       mode="sigmoid", bias=conv["bias"], n_groups=4, topk_groups=2, renorm=True, scale=2.5,
                       shared=conv["shared"])
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    xd = x.to(dev)
    out, logits, w, ids = pkg.layer_fp8(xd, conv["router_weight"], conv["w13"], conv["w13_scale"], conv["w2"],
                                        conv["w2_scale"], K, "sigmoid", bias=conv["bias"], n_groups=4, topk_groups=2,
                                        renorm=True, scale=2.5, shared=conv["shared"], return_routing=True)
    assert torch.equal(moe(xd).view(torch.int16), out.view(torch.int16))
    torch.cuda.synchronize()
    # the oracle on the checkpoint's own per-expert tensors (nothing of the converter is reused)
    stack = lambda proj: (torch.stack([per_expert[(e, proj)][0] for e in range(E)]),
                          torch.stack([per_expert[(e, proj)][1] for e in range(E)]))
    (gq, gs), (uq, us), (dq, ds) = stack("gate_proj"), stack("up_proj"), stack("down_proj")
    layer = (torch.cat([gq, uq], 1), torch.cat([gs, us], 1), dq, ds)
    sh = (torch.cat([per_expert[("s", "gate_proj")][0], per_expert[("s", "up_proj")][0]], 0)[None],
          torch.cat([per_expert[("s", "gate_proj")][1], per_expert[("s", "up_proj")][1]], 0)[None],
          per_expert[("s", "down_proj")][0][None], per_expert[("s", "down_proj")][1][None])
    scores = pkg.moe_route(logits, K, "sigmoid", bias=conv["bias"], n_groups=4, topk_groups=2, renorm=True, scale=2.5,
                           return_scores=True)[2].cpu()
    w_ref, ids_ref = oracle.select_sigmoid_grouped(scores, state[pre + "gate.e_score_correction_bias"], K, 4, 2, 2.5, True)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    ref = oracle.moe_w8a8_fp32(x, ids_ref, w_ref, *layer, shared=sh)
    got = out.float().cpu()
    assert checks.outside_fraction(got, ref) <= checks.MAX_OUTSIDE
    assert oracle.cal_diff(ref, got)[0] < 1e-5
    # the converter's packed bytes are the oracle's row-major tensors, tile-blocked
    assert torch.equal(pkg.unpack_weights(conv["w13"]).cpu().view(torch.uint8), layer[0].view(torch.uint8))
    assert torch.equal(pkg.unpack_weights(conv["w2"]).cpu().view(torch.uint8), layer[2].view(torch.uint8))
    rep = checks.check_sample(pkg, oracle, xd, ids, (conv["w13"], conv["w13_scale"], conv["w2"], conv["w2_scale"]),
                              w_s=w, shared_dev=conv["shared"], out_big=out, what="converted checkpoint")
    say("   ", rep)
    # the reference's argument form of the same weights: pre-transposed down, bf16-representable scales aside, the
    # packed bytes are identical
    packed = pkg.pack_expert_weights(gq.to(dev), uq.to(dev), dq.transpose(1, 2).contiguous().to(dev), gs.to(dev),
                                     us.to(dev), ds.transpose(1, 2).contiguous().to(dev))
    torch.cuda.synchronize()
    for a, b in zip(packed, (conv["w13"], conv["w13_scale"], conv["w2"], conv["w2_scale"])):
        assert torch.equal(a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a,
                           b.view(torch.uint8) if b.dtype == torch.float8_e4m3fn else b)
    # and the registered op form of the same packing
    packed2 = torch.ops.my_ops.moe_pack_weights(gq.to(dev), uq.to(dev), dq.transpose(1, 2).contiguous().to(dev), gs.to(dev),
                                                us.to(dev), ds.transpose(1, 2).contiguous().to(dev))
    assert all(torch.equal(a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a,
                           b.view(torch.uint8) if b.dtype == torch.float8_e4m3fn else b) for a, b in zip(packed, packed2))
    # the router op and the permutation op of the same namespace
    w_op, ids_op = torch.ops.my_ops.moe_route(xd, conv["router_weight"], conv["bias"], "sigmoid", K, 4, 2, 2.5, True)
    assert torch.equal(ids_op, ids) and torch.equal(w_op, w)
    ss, off, s2r = torch.ops.my_ops.moe_permute(ids, E)
    ss_ref, off_ref, s2r_ref = oracle.permute_counting_sort(ids.cpu(), E)
    assert torch.equal(ss.cpu(), ss_ref) and torch.equal(off.cpu(), off_ref) and torch.equal(s2r.cpu(), s2r_ref)


def test_checkpoint_converter_pads_ragged_sizes_and_names_the_device_it_needs(pkg, oracle, dev):
    """A checkpoint whose H and I are no multiples of 128 (partial blocks at the edges, ceil(n/128) scales): the
    converter pads codes to whole blocks like the reference-layout packer does, and the layer runs on activations
    padded the same way; asked to tile-block host tensors it says what it needs."""
    say("checkpoint converter, ragged sizes")
    E, H, I, K, T = 4, 328, 200, 2, 9
    Hp, Ip = 384, 256
    g = torch.Generator().manual_seed(5)
    state, pre = {}, "m."
    dense = {}
    for e in range(E):
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            wfull = torch.zeros(-(-n // 128) * 128, -(-k // 128) * 128)
            wfull[:n, :k] = torch.randn(n, k, generator=g) * 0.05
            q, sc = oracle.quant_weight_block128(wfull)
            state[f"{pre}experts.{e}.{proj}.weight"], state[f"{pre}experts.{e}.{proj}.weight_scale_inv"] = q[:n, :k].contiguous(), sc
            dense[(e, proj)] = (q, sc)
    state[pre + "gate.weight"] = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="device="):
        pkg.convert_hf_moe_layer(state, pre, E)
    conv = pkg.convert_hf_moe_layer(state, pre, E, device=dev)
    assert tuple(conv["w13"].shape) == (E, 2 * Ip, Hp) and tuple(conv["w2"].shape) == (E, Hp, Ip)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    xp = torch.nn.functional.pad(x, (0, Hp - H)).to(dev)
    ids, w = torch.tensor([[e % E, (e + 1) % E] for e in range(T)], dtype=torch.int32), torch.full((T, K), 0.5)
    out = pkg.fused_experts_fp8(xp, conv["w13"], conv["w13_scale"], conv["w2"], conv["w2_scale"], ids.to(dev), w.to(dev))
    torch.cuda.synchronize()
    layer = (torch.cat([torch.stack([dense[(e, "gate_proj")][0] for e in range(E)]),
                        torch.stack([dense[(e, "up_proj")][0] for e in range(E)])], 1),
             torch.cat([torch.stack([dense[(e, "gate_proj")][1] for e in range(E)]),
                        torch.stack([dense[(e, "up_proj")][1] for e in range(E)])], 1),
             torch.stack([dense[(e, "down_proj")][0] for e in range(E)]),
             torch.stack([dense[(e, "down_proj")][1] for e in range(E)]))
    ref = oracle.moe_w8a8_fp32(xp.cpu(), ids, w, *layer)
    got = out.float().cpu()
    assert float(got[:, H:].abs().max()) == 0.0            # the padding columns of the output are zero
    scale = ref.abs().max().item()
    assert ((got - ref).abs() <= 1e-2 * scale + 2e-2 * ref.abs()).float().mean() >= 0.995


@pytest.mark.parametrize("T,E,K,mode,G,TG", [(1, 384, 8, "sigmoid", 8, 4), (9, 512, 6, "softmax", 1, 1),
                                             (40, 1024, 8, "sigmoid", 16, 5), (300, 320, 4, "softmax_logit_bias", 1, 1)])
def test_layer_entry_point_with_more_than_256_experts(pkg, oracle, dev, checks, T, E, K, mode, G, TG):
    """Layers with more than 256 experts (up to 1024) run behind the same entry point: the router product in blocks of
    256 experts, routing from the partial sums, the permutation.  Logits against an fp64 product; ids and weights equal
    the stand-alone routing entry point's on the same logits and the oracle's; the output equals the staged entry
    point's on the same routing, bit for bit; a sample of tokens through the strict steps."""
    say("layer with", E, "experts, T =", T, mode)
    H, I = 512, 128
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=E)))
    g = torch.Generator().manual_seed(E + T)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bias = None if mode == "softmax" else (torch.randn(E, generator=g) * 0.1).to(dev)
    scale = 2.5 if mode == "sigmoid" else 1.0
    out, logits, w, ids = pkg.layer_fp8(x, wr, *ld, K, mode, bias=bias, n_groups=G, topk_groups=TG, renorm=True, scale=scale,
                                        return_routing=True)
    torch.cuda.synchronize()
    exact = x.double().cpu() @ wr.double().cpu().t()
    err = (logits.double().cpu() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4 * x.double().cpu().norm(dim=1, keepdim=True) * wr.double().cpu().norm(dim=1)[None]
    assert bool((err <= bound).all())
    assert torch.equal(logits.view(torch.int16), pkg.router_logits(x, wr).view(torch.int16))
    w1, ids1 = pkg.moe_route(logits, K, mode, bias=bias, n_groups=G, topk_groups=TG, renorm=True, scale=scale)
    assert torch.equal(ids, ids1) and torch.equal(w, w1)
    if mode == "sigmoid":
        scores = pkg.moe_route(logits, K, mode, bias=bias, n_groups=G, topk_groups=TG, renorm=True, scale=scale,
                               return_scores=True)[2].cpu()
        w_ref, ids_ref = oracle.select_sigmoid_grouped(scores, bias.cpu(), K, G, TG, scale, True)
    else:
        lg = logits.float().cpu() + (bias.cpu() if mode == "softmax_logit_bias" else 0.0)
        w_ref, ids_ref = oracle.route_softmax_topk(lg, K, True)
    assert torch.equal(ids.cpu(), ids_ref) and torch.allclose(w.cpu(), w_ref, rtol=1e-5, atol=1e-7)
    staged = pkg.fused_experts_fp8(x, *ld, ids, w)
    assert torch.equal(out.view(torch.int16), staged.view(torch.int16))
    moe = pkg.FusedMoE(wr, *ld, top_k=K, mode="softmax" if mode == "softmax_logit_bias" else mode, bias=bias, n_groups=G,
                       topk_groups=TG, renorm=True, scale=scale)
    assert torch.equal(moe(x).view(torch.int16), out.view(torch.int16))
    wm, im = moe.route(x)                                  # the module's staged road: the same kernels, call by call
    assert torch.equal(im, ids) and torch.equal(wm, w)
    pick = torch.arange(min(T, 6), device=dev)
    rep = checks.check_sample(pkg, oracle, x[pick].contiguous(), ids[pick].contiguous(), ld, w_s=w[pick].contiguous(),
                              out_big=out[pick].contiguous(), what=f"E={E}")
    say("   ", rep)


def test_module_form_holds_its_weights_as_buffers(pkg, oracle, dev):
    """FusedMoEModule: the nn.Module shape the reference's tests give their wrapper (test_moe.py:143-160).  Its buffers
    travel through state_dict / load_state_dict, and forward equals the plain class bit for bit."""
    say("nn.Module form")
    T, H, I, E, K = 20, 512, 256, 16, 4
    ld = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=3)))
    sh = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(1, H, I, seed=4)))
    g = torch.Generator().manual_seed(8)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(dev)                          # fp32: rounded to bf16 once
    bias = (torch.randn(E, generator=g) * 0.1).to(dev)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    mod = pkg.FusedMoEModule(wr, *ld, top_k=K, mode="sigmoid", bias=bias, n_groups=4, topk_groups=2, scale=2.5, shared=sh)
    ref = pkg.FusedMoE(wr, *ld, top_k=K, mode="sigmoid", bias=bias, n_groups=4, topk_groups=2, scale=2.5, shared=sh)
    out = mod(x)
    assert torch.equal(out.view(torch.int16), ref(x).view(torch.int16))
    state = mod.state_dict()
    assert {"router_weight", "w13", "w13_scale", "w2", "w2_scale", "bias", "shared_w13", "shared_w2"} <= set(state)
    other = pkg.FusedMoEModule(torch.zeros_like(wr), *(torch.zeros_like(t) for t in ld), top_k=K, mode="sigmoid",
                               bias=torch.zeros_like(bias), n_groups=4, topk_groups=2, scale=2.5,
                               shared=tuple(torch.zeros_like(t) for t in sh))
    other.load_state_dict(state)
    assert torch.equal(other(x).view(torch.int16), out.view(torch.int16))
