"""GPU parity of the dense block-scaled FP8 layers (my_ops.mm_w8a16_dq_forward, mlp_w8a16_dq_forward)
against the oracle, on the reference's own shape grids and data recipes
(python/regression/test_llm/test_mm_w8a16_dq.py:101-109, test_deepseek_mm.py:125-132,194-200,
test_mlp_w8a16_dq.py:141-148: x ~ N(0,1) bf16, weights N(0,1) cast to e4m3fn, scales N(0,1) bf16)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-2          # on outputs normalised to unit rms
MAX_OUTSIDE = 5e-3               # MLP only: share of elements a one-step flip of a re-quantised code may move


def say(*a):
    print(*a, flush=True)


def normalised_outside(got, ref):
    rms = ref.pow(2).mean().sqrt().clamp_min(1e-12)
    g, r = got / rms, ref / rms
    return ((g - r).abs() > ATOL + RTOL * r.abs()).float().mean().item()


MM_SHAPES = [(32, 7168, 1536), (32, 7168, 576), (32, 2048, 7168), (64, 4096, 2048), (128, 7168, 1536),
             (256, 4096, 1024), (1, 256, 16), (200, 384, 272), (100, 4096, 8192), (128, 1024, 64),
             # few rows, wide layer or short reduction: the grouped kernels' strips instead of the per-wavefront kernel
             (32, 4096, 14336), (1, 2304, 12288), (128, 1024, 16384), (17, 7168, 12288), (64, 2048, 7168),
             # more than 128 rows of a narrow layer under a long reduction: the per-wavefront kernel, several row chunks
             (256, 7168, 1536), (384, 16384, 1024), (512, 7168, 512), (385, 7168, 1536), (513, 7168, 512)]


@pytest.mark.parametrize("M,K,N", MM_SHAPES)
def test_mm_w8a16_dq_forward(pkg, oracle, dev, M, K, N):
    say("mm", M, K, N)
    g = torch.Generator().manual_seed(1000 + M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    s = torch.randn((N + 127) // 128, K // 128, generator=g).to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    r = torch.ops.my_ops.mm_w8a16_dq_forward(x.to(dev), w.to(dev), s.to(dev), out, 128)
    torch.cuda.synchronize()
    assert r.data_ptr() == out.data_ptr()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    # the reference's criterion against its own bf16 ground truth
    assert oracle.cos_sim(oracle.mm_w8a16_dq_ref(x, w, s).float().flatten(), got.flatten()) >= 0.99
    # the same quantised operands multiplied in fp32: every element within tolerance
    ref = oracle.mm_w8a8_fp32(x, w, s.float())
    assert normalised_outside(got, ref) == 0.0


@pytest.mark.parametrize("M,H,I", [(32, 7168, 2304), (32, 7168, 256), (64, 4096, 2048), (1, 256, 128), (200, 512, 384),
                                   (32, 4096, 8192), (100, 1024, 1024)])
def test_mlp_w8a16_dq_forward(pkg, oracle, dev, M, H, I):
    say("mlp", M, H, I)
    g = torch.Generator().manual_seed(2000 + M + I)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    wg = torch.randn(I, H, generator=g).to(torch.float8_e4m3fn)
    wu = torch.randn(I, H, generator=g).to(torch.float8_e4m3fn)
    wd = torch.randn(H, I, generator=g).to(torch.float8_e4m3fn)
    sg = torch.randn(I // 128, H // 128, generator=g).to(torch.bfloat16)
    su = torch.randn(I // 128, H // 128, generator=g).to(torch.bfloat16)
    sd = torch.randn(H // 128, I // 128, generator=g).to(torch.bfloat16)
    out = torch.empty(M, H, dtype=torch.bfloat16, device=dev)
    # the reference hands the down projection and its scales over transposed (non-contiguous views)
    torch.ops.my_ops.mlp_w8a16_dq_forward(x.to(dev), wg.to(dev), wu.to(dev), wd.T.to(dev), sg.to(dev), su.to(dev),
                                          sd.T.to(dev), out, 128)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert oracle.cos_sim(oracle.mlp_w8a16_dq_ref(x, wg, wu, wd, sg, su, sd).float().flatten(), got.flatten()) >= 0.99
    w13q, w13s = torch.cat([wg, wu], 0), torch.cat([sg, su], 0).float()
    ref, mid = oracle.mlp_w8a8_fp32(x, w13q, w13s, wd, sd.float(), return_mid=True)
    assert normalised_outside(got, ref) <= MAX_OUTSIDE
    assert oracle.cal_diff(ref, got)[0] < 1e-4


@pytest.mark.parametrize("block", [64, 256])
@pytest.mark.parametrize("M,K,N", [(32, 2048, 512), (16, 2048, 512), (200, 1024, 272), (40, 1000, 100), (3, 72, 7)])
def test_mm_block_sizes(pkg, oracle, dev, M, K, N, block):
    """The reference's block-size grid (python/regression/test_llm/test_deepseek_mm.py:225-248: 64, 128, 256 on
    32 x 2048 -> 512).  256: the FP8 kernels on scales expanded to 128-blocks; 64: the reference's bf16 arithmetic."""
    say("mm block", block, M, K, N)
    g = torch.Generator().manual_seed(3000 + block + M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    s = torch.rand((N + block - 1) // block, (K + block - 1) // block, generator=g).to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.mm_w8a16_dq_forward(x.to(dev), w.to(dev), s.to(dev), out, block)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref16 = oracle.mm_w8a16_dq_ref(x, w, s, block).float()
    assert oracle.cos_sim(ref16.flatten(), got.flatten()) >= 0.99
    if block == 64:
        # same arithmetic as the reference: bf16 operands, fp32 accumulation, one rounding
        ref = x.float() @ oracle.weight_dequant_literal(w, s, block).float().T
        assert normalised_outside(got, ref) == 0.0
        assert oracle.cal_diff(ref16, got)[0] < 1e-4
    else:
        xq, xs = oracle.act_quant_group128(x)
        ref = oracle.act_dequant_group128(xq, xs) @ oracle.dequant_block(w, s.float(), block).T
        assert normalised_outside(got, ref) == 0.0


@pytest.mark.parametrize("block", [64, 256])
def test_mlp_block_sizes(pkg, oracle, dev, block):
    say("mlp block", block)
    M, H, I = 48, 512, 256
    g = torch.Generator().manual_seed(4000 + block)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    wg, wu = (torch.randn(I, H, generator=g).to(torch.float8_e4m3fn) for _ in range(2))
    wd = torch.randn(H, I, generator=g).to(torch.float8_e4m3fn)
    sg, su = (torch.rand(I // block, H // block, generator=g).mul(0.1).to(torch.bfloat16) for _ in range(2))
    sd = torch.rand(H // block, I // block, generator=g).mul(0.1).to(torch.bfloat16)
    out = torch.empty(M, H, dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.mlp_w8a16_dq_forward(x.to(dev), wg.to(dev), wu.to(dev), wd.T.to(dev), sg.to(dev), su.to(dev),
                                          sd.T.to(dev), out, block)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref16 = oracle.mlp_w8a16_dq_ref(x, wg, wu, wd, sg, su, sd, block).float()
    assert oracle.cos_sim(ref16.flatten(), got.flatten()) >= 0.99
    if block == 64:
        assert oracle.cal_diff(ref16, got)[0] < 1e-4
        assert normalised_outside(got, ref16) <= MAX_OUTSIDE
    else:
        w13q = torch.cat([wg, wu], 0)
        w13s = torch.cat([sg, su], 0).float().repeat_interleave(2, 0).repeat_interleave(2, 1)
        ref = oracle.mlp_w8a8_fp32(x, w13q, w13s, wd, sd.float().repeat_interleave(2, 0).repeat_interleave(2, 1))
        assert normalised_outside(got, ref) <= MAX_OUTSIDE
        assert oracle.cal_diff(ref, got)[0] < 1e-4


def test_dense_ops_reject_what_they_do_not_support(pkg, dev):
    x = torch.zeros(4, 256, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(128, 256, dtype=torch.float8_e4m3fn, device=dev)
    s = torch.ones(1, 2, dtype=torch.bfloat16, device=dev)
    out = torch.empty(4, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        torch.ops.my_ops.mm_w8a16_dq_forward(x, w, s, out, 0)
    with pytest.raises(RuntimeError):
        torch.ops.my_ops.mm_w8a16_dq_forward(x, w.view(torch.uint8), s, out, 128)


@pytest.mark.parametrize("M,K,N", [(32, 7168, 1536), (1, 256, 16), (200, 384, 272), (100, 4096, 8192), (300, 1024, 2048)])
def test_mm_in_the_references_own_arithmetic(pkg, oracle, dev, M, K, N):
    """set_expert_numerics('w8a16'): mm_w8a16_dq_forward multiplies bf16 activations with weights de-quantised in
    registers (MmW8A16Dq.cpp:185-228); against the reference's bf16 ground truth
    (python/regression/test_llm/test_mm_w8a16_dq.py:52-60) cos_diff < 1e-4, which the FP8-activation path cannot reach."""
    say("mm w8a16", M, K, N)
    g = torch.Generator().manual_seed(3000 + M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    s = torch.randn((N + 127) // 128, K // 128, generator=g).to(torch.bfloat16)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.set_expert_numerics("w8a16")
    try:
        torch.ops.my_ops.mm_w8a16_dq_forward(x.to(dev), w.to(dev), s.to(dev), out, 128)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref = oracle.mm_w8a16_dq_ref(x, w, s).float()
    assert oracle.cos_sim(ref.flatten(), got.flatten()) >= 0.99
    assert oracle.cal_diff(ref, got)[0] < 1e-4
    # element-wise: one bf16 rounding of an fp32 sum against the reference's bf16 matmul
    rms = ref.pow(2).mean().sqrt()
    assert ((got - ref).abs() <= 1.6e-2 * ref.abs() + 1e-2 * rms).all()


@pytest.mark.parametrize("M,H,I", [(32, 7168, 256), (1, 256, 128), (200, 512, 384), (300, 1024, 1024)])
def test_mlp_in_the_references_own_arithmetic(pkg, oracle, dev, M, H, I):
    """The gated MLP likewise (MlpW8A16Dq.cpp:189-241; python/regression/test_llm/test_mlp_w8a16_dq.py:53-81)."""
    say("mlp w8a16", M, H, I)
    g = torch.Generator().manual_seed(4000 + M + I)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    wg, wu = (torch.randn(I, H, generator=g).to(torch.float8_e4m3fn) for _ in range(2))
    wd = torch.randn(H, I, generator=g).to(torch.float8_e4m3fn)
    sg, su = ((torch.randn(I // 128, H // 128, generator=g) * 0.05).to(torch.bfloat16) for _ in range(2))
    sd = (torch.randn(H // 128, I // 128, generator=g) * 0.05).to(torch.bfloat16)
    out = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.set_expert_numerics("w8a16")
    try:
        torch.ops.my_ops.mlp_w8a16_dq_forward(x.to(dev), wg.to(dev), wu.to(dev), wd.T.to(dev), sg.to(dev), su.to(dev),
                                              sd.T.to(dev), out, 128)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref = oracle.mlp_w8a16_dq_ref(x, wg, wu, wd, sg, su, sd).float()
    assert oracle.cos_sim(ref.flatten(), got.flatten()) >= 0.99
    assert oracle.cal_diff(ref, got)[0] < 1e-4


@pytest.mark.parametrize("seed", range(20))
def test_mm_random_shapes_both_arithmetics(pkg, oracle, dev, seed):
    """mm_w8a16_dq_forward on shapes drawn from the seed: row counts either side of the 128 rows up to which the
    per-wavefront kernel runs, output widths of any size, reductions of 1 to 56 blocks or with a partial last block; FP8
    activations strict against the fp32 product of the same quantised operands, the reference's own arithmetic against
    its bf16 ground truth at its criterion (python/regression/test_llm/test_mm_w8a16_dq.py:52-60)."""
    import random
    r = random.Random(4000 + seed)
    M = r.choice([1, 2, 7, 16, 31, 64, 127, 128, 129, 200, 333])
    K = r.choice([128 * r.choice([1, 2, 3, 8, 16, 33, 56]), 128 * r.choice([1, 2, 3, 8, 16, 33, 56]), 8 * r.randint(1, 150)])
    N = r.choice([16 * r.randint(1, 40), 128 * r.randint(1, 24), 8 * r.randint(2, 90), r.randint(1, 300)])
    say("mm random", seed, M, K, N)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    s = (torch.rand((N + 127) // 128, (K + 127) // 128, generator=g) + 0.1).to(torch.bfloat16)
    xd, wd, sd = x.to(dev), w.to(dev), s.to(dev)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.mm_w8a16_dq_forward(xd, wd, sd, out, 128)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert normalised_outside(got, oracle.mm_w8a8_fp32(x, w, s.float())) == 0.0
    out16 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.set_expert_numerics("w8a16")
    try:
        torch.ops.my_ops.mm_w8a16_dq_forward(xd, wd, sd, out16, 128)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got16 = out16.float().cpu()
    ref = oracle.mm_w8a16_dq_ref(x, w, s).float()
    assert torch.isfinite(got16).all()
    assert oracle.cos_sim(ref.flatten(), got16.flatten()) >= 0.99
    assert oracle.cal_diff(ref, got16)[0] < 1e-4
    rms = ref.pow(2).mean().sqrt()
    assert ((got16 - ref).abs() <= 1.6e-2 * ref.abs() + 1e-2 * rms).all()


@pytest.mark.parametrize("seed", range(12))
def test_mlp_random_shapes_both_arithmetics(pkg, oracle, dev, seed):
    """mlp_w8a16_dq_forward on shapes drawn from the seed, hidden and intermediate sizes that 128 may not divide
    (torch_tpu/csrc/ops/my_ops/MlpW8A16Dq.pl:11-34 takes ceil(n/128) blocks): the reference's own arithmetic against its
    ground truth at its criterion (python/regression/test_llm/test_mlp_w8a16_dq.py:53-81), the FP8 activation path
    against the fp32 computation on the same quantised operands."""
    import random
    r = random.Random(5000 + seed)
    M = r.choice([1, 5, 16, 33, 64, 127, 129, 250])
    H = r.choice([128 * r.randint(1, 16), 8 * r.randint(4, 150)])
    I = r.choice([128 * r.randint(1, 8), 8 * r.randint(4, 100)])
    say("mlp random", seed, M, H, I)
    g = torch.Generator().manual_seed(seed)
    nb = lambda n: (n + 127) // 128
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    wg, wu = (torch.randn(I, H, generator=g).to(torch.float8_e4m3fn) for _ in range(2))
    wd = torch.randn(H, I, generator=g).to(torch.float8_e4m3fn)
    sg, su = ((torch.rand(nb(I), nb(H), generator=g) * 0.05 + 0.005).to(torch.bfloat16) for _ in range(2))
    sd = (torch.rand(nb(H), nb(I), generator=g) * 0.05 + 0.005).to(torch.bfloat16)
    args = (x.to(dev), wg.to(dev), wu.to(dev), wd.T.to(dev), sg.to(dev), su.to(dev), sd.T.to(dev))
    out = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.mlp_w8a16_dq_forward(*args, out, 128)
    out16 = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
    pkg.set_expert_numerics("w8a16")
    try:
        torch.ops.my_ops.mlp_w8a16_dq_forward(*args, out16, 128)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    got, got16 = out.float().cpu(), out16.float().cpu()
    assert torch.isfinite(got).all() and torch.isfinite(got16).all()
    truth = oracle.mlp_w8a16_dq_ref(x, wg, wu, wd, sg, su, sd).float()
    assert oracle.cos_sim(truth.flatten(), got16.flatten()) >= 0.99
    assert oracle.cal_diff(truth, got16)[0] < 1e-4
    assert oracle.cos_sim(truth.flatten(), got.flatten()) >= 0.99
    # the FP8 path against fp32 arithmetic on the same quantised operands, ragged sizes padded with zeros as the device does
    Hp, Ip = nb(H) * 128, nb(I) * 128
    pad = lambda t, rows, cols: torch.nn.functional.pad(t.view(torch.uint8), (0, cols - t.shape[1], 0, rows - t.shape[0])).view(t.dtype)
    w13q = torch.cat([pad(wg, Ip, Hp), pad(wu, Ip, Hp)], 0)
    ref = oracle.mlp_w8a8_fp32(torch.nn.functional.pad(x, (0, Hp - H)), w13q, torch.cat([sg, su], 0).float(),
                               pad(wd, Hp, Ip), sd.float())[:, :H]
    assert normalised_outside(got, ref) <= MAX_OUTSIDE
    assert oracle.cal_diff(ref, got)[0] < 1e-4


@pytest.mark.parametrize("M,H,I", [(32, 7168, 256), (200, 512, 384), (5, 328, 200)])
def test_mlp_w8a8_quant_forward(pkg, oracle, dev, M, H, I):
    """mlp_w8a8_quant_forward (torch_tpu/csrc/ops/my_ops/MlpW8A8Quant.cpp:12-52): the FP8-activation arithmetic whatever
    the numerics switch says, the down projection in either orientation (the W8A16 op's transposed one, or [H, I] as
    python/test/deepseek_mlp_quant.py:167-177 builds it), against fp32 arithmetic on the same quantised operands.  The
    reference pins nothing for this op (closed implementation, no test, no CPU function): the comparison is with this
    package's own definition of the activation quantisation."""
    say("mlp w8a8", M, H, I)
    g = torch.Generator().manual_seed(6000 + M + I)
    nb = lambda n: (n + 127) // 128
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    wg, wu = (torch.randn(I, H, generator=g).to(torch.float8_e4m3fn) for _ in range(2))
    wd = torch.randn(H, I, generator=g).to(torch.float8_e4m3fn)
    sg, su = ((torch.rand(nb(I), nb(H), generator=g) * 0.05 + 0.005).to(torch.bfloat16) for _ in range(2))
    sd = (torch.rand(nb(H), nb(I), generator=g) * 0.05 + 0.005).to(torch.bfloat16)
    xd, wgd, wud, wdd, sgd, sud, sdd = (t.to(dev) for t in (x, wg, wu, wd, sg, su, sd))
    wdt, sdt = wdd.T.contiguous(), sdd.T.contiguous()
    base = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
    torch.ops.my_ops.mlp_w8a16_dq_forward(xd, wgd, wud, wdt, sgd, sud, sdt, base, 128)       # default numerics: FP8 activations
    outs = []
    pkg.set_expert_numerics("w8a16")
    try:
        for down, scale in ((wdt, sdt), (wdd, sdd)):
            out = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=dev)
            r = torch.ops.my_ops.mlp_w8a8_quant_forward(xd, wgd, wud, down, sgd, sud, scale, out, 128)
            assert r.data_ptr() == out.data_ptr()
            outs.append(out)
        torch.cuda.synchronize()
    finally:
        pkg.set_expert_numerics("w8a8")
    for out in outs:
        assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    got = base.float().cpu()
    Hp, Ip = nb(H) * 128, nb(I) * 128
    pad = lambda t, rows, cols: torch.nn.functional.pad(t.view(torch.uint8), (0, cols - t.shape[1], 0, rows - t.shape[0])).view(t.dtype)
    ref = oracle.mlp_w8a8_fp32(torch.nn.functional.pad(x, (0, Hp - H)), torch.cat([pad(wg, Ip, Hp), pad(wu, Ip, Hp)], 0),
                               torch.cat([sg, su], 0).float(), pad(wd, Hp, Ip), sd.float())[:, :H]
    assert normalised_outside(got, ref) <= MAX_OUTSIDE
    assert oracle.cal_diff(ref, got)[0] < 1e-4


def test_w8a16_beyond_its_range_raises_instead_of_switching_arithmetic(pkg, dev):
    """set_expert_numerics('w8a16') covers reduction lengths up to 16384.  Beyond that the dense ops (and the expert op)
    raise; they never fall through to the FP8-activation arithmetic the caller did not select."""
    M, K, N = 4, 16384 + 128, 32
    w = torch.zeros(N, K, dtype=torch.float8_e4m3fn, device=dev)
    s = torch.ones(N // 128 + 1, K // 128, dtype=torch.bfloat16, device=dev)
    x = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    pkg.set_expert_numerics("w8a16")
    try:
        with pytest.raises(RuntimeError, match="up to 16384"):
            torch.ops.my_ops.mm_w8a16_dq_forward(x, w, s, out, 128)
    finally:
        pkg.set_expert_numerics("w8a8")
    torch.ops.my_ops.mm_w8a16_dq_forward(x, w, s, out, 128)        # the default arithmetic takes the shape
    torch.cuda.synchronize()
    assert float(out.float().abs().max()) == 0.0
