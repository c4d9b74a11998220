"""The C-ABI library without a GPU: it loads, exports every symbol the header declares, and
rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "moe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for s in ["moe_fused_experts_fp8", "moe_noaux_tc_topk", "moe_route_topk", "moe_permute", "moe_scale_pitch", "moe_act_quant",
              "moe_gemm1_swiglu", "moe_gemm2", "moe_weighted_reduce", "moe_hip_version"]:
        assert s in syms


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(os.path.join(ROOT, "torch-tpu_amd", "libmoe_hip.so"))
    for s in declared_symbols():
        assert hasattr(lib, s), f"{s} is declared in include/moe_hip.h but not exported"


def test_binding_table_covers_the_header(pkg):
    from torch_tpu_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_version_and_arch(pkg):
    from torch_tpu_amd._lib import lib
    assert lib.moe_hip_version() >= 200      # 200: tile-blocked weights
    assert lib.moe_hip_arch() == b"gfx950"
    assert lib.moe_hip_strerror(0) == b"ok"
    assert b"NULL" in lib.moe_hip_strerror(-1)


def test_argument_errors_are_codes_not_crashes(pkg):
    from torch_tpu_amd._lib import lib
    E_NULL, E_SHAPE, E_ALIGN, E_WS, E_MODE = -1, -2, -3, -4, -5
    fake = ctypes.c_void_p(0x1000)          # never dereferenced: validation fails first
    assert lib.moe_act_quant(None, None, 4, 128, fake, fake) == E_NULL
    assert lib.moe_act_quant(None, fake, 4, 100, fake, fake) == E_ALIGN
    assert lib.moe_noaux_tc_topk(None, fake, 7, 1, 256, 8, 4, 8, fake, fake) == E_MODE
    assert lib.moe_noaux_tc_topk(None, fake, 0, 1, 250, 8, 4, 8, fake, fake) == E_SHAPE      # 250 % 8 != 0
    assert lib.moe_noaux_tc_topk(None, fake, 0, 1, 4096, 8, 4, 8, fake, fake) == E_SHAPE     # too many experts
    assert lib.moe_route_topk(None, fake, 0, None, 1, 8, 9, 0, 1, 1, 1, 1.0, fake, fake, None) == E_SHAPE
    assert lib.moe_route_topk(None, fake, 0, None, 1, 8, 2, 9, 1, 1, 1, 1.0, fake, fake, None) == E_MODE
    assert lib.moe_permute(None, fake, 4, 2, 8, fake, fake, fake, fake, 16) == E_WS
    assert lib.moe_mm_fp8(None, fake, 4, 200, fake, fake, 64, fake, fake, 1 << 20) == E_ALIGN    # K % 128
    assert lib.moe_mm_fp8(None, fake, 4, 256, fake, fake, 8, fake, fake, 1 << 20) == E_SHAPE     # N < 16
    assert lib.moe_mlp_fp8(None, fake, 4, 256, fake, fake, fake, fake, 128, fake, fake, 16) == E_WS
    # reduction lengths beyond 32768 and activation tensors of 2 GiB or more are refused before anything is launched
    big = [None, fake, 4, 65536, fake, fake, fake, fake, 128, 8, fake, fake, 2, None, None, None, None, 0, fake, 1, fake, 1 << 40]
    assert lib.moe_fused_experts_fp8(*big) == E_SHAPE
    big[2], big[3] = 400000, 7168
    assert lib.moe_fused_experts_fp8(*big) == E_SHAPE
    assert lib.moe_mm_bf16(None, fake, 4, 200, fake, 64, fake) == E_ALIGN                        # K % 64
    assert lib.moe_mm_bf16(None, fake, 4, 32768, fake, 64, fake) == E_SHAPE                      # K > 16384
    assert lib.moe_mm_bf16(None, fake, 4, 256, None, 64, fake) == E_NULL
    assert lib.moe_mm_bf16(None, None, 0, 256, fake, 64, None) == 0                              # no rows: nothing to do
    assert lib.moe_permute(None, fake, 4, 2, 5000, fake, fake, fake, fake, 1 << 20) == E_SHAPE
    ws = lib.moe_fused_experts_workspace_bytes(4, 256, 512, 8, 2, 0)
    assert ws > 0 and ws % 256 == 0
    args = dict(T=4, H=256, I=512, E=8, K=2)

    def fused(x=fake, H=256, I=512, out_mode=0, wsb=ws, rw=None, workspace=fake):
        return lib.moe_fused_experts_fp8(None, x, 4, H, fake, fake, fake, fake, I, 8, fake, rw, 2,
                                         None, None, None, None, 0, fake, out_mode, workspace, wsb)
    assert fused(x=None) == E_NULL
    assert fused(H=200) == E_ALIGN
    assert fused(I=100) == E_ALIGN
    assert fused(out_mode=3) == E_MODE
    assert fused(out_mode=1) == E_NULL            # weighted output needs routing weights
    assert fused(wsb=ws - 1) == E_WS
    assert fused(workspace=ctypes.c_void_p(0x1004)) == E_ALIGN
    del args


def test_workspace_sizes_grow_with_the_problem(pkg):
    from torch_tpu_amd._lib import lib
    small = lib.moe_fused_experts_workspace_bytes(16, 256, 512, 8, 2, 0)
    big = lib.moe_fused_experts_workspace_bytes(4096, 7168, 2048, 256, 8, 2048)
    assert 0 < small < big
    # the big pieces: y [T*K, H] bf16 + hq [T*K, I] + xq [T, H]
    assert big >= 4096 * 8 * 7168 * 2 + 4096 * 8 * 2048 + 4096 * 7168
    assert lib.moe_permute_workspace_bytes(4096, 8, 256) >= (4096 * 8 // 256) * 256 * 4
    for T in (1, 16, 17, 32, 33, 64, 65, 4096):
        assert lib.moe_tile_rows(T, 8, 256) in (16, 32, 64, 128, 192)


def test_python_wrappers_validate_before_launch(pkg):
    import torch
    x = torch.zeros(4, 256, dtype=torch.bfloat16)          # CPU tensor: must be refused
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.act_quant(x)
    with pytest.raises(RuntimeError, match="int32"):
        pkg.noaux_tc_topk(torch.zeros(1, 8), torch.zeros(1, 8, dtype=torch.int64), torch.zeros(1, 256), 8, 4, 8)
    with pytest.raises(RuntimeError, match="same dtype"):
        pkg.noaux_tc_topk(torch.zeros(1, 8, dtype=torch.bfloat16), torch.zeros(1, 8, dtype=torch.int32),
                          torch.zeros(1, 256), 8, 4, 8)


def test_my_ops_are_registered_with_reference_arity(pkg):
    import torch
    ops = torch.ops.my_ops
    assert len(ops.fused_moe_fused_experts.default._schema.arguments) == 25
    assert len(ops.fused_moe_fused_experts_v2.default._schema.arguments) == 27
    assert len(ops.noaux_tc_topk.default._schema.arguments) == 6
    assert len(ops.fused_moe_grouped_topk.default._schema.arguments) == 10
    assert len(ops.mlp_w8a16_dq_forward.default._schema.arguments) == 9     # ops.hpp:279-288
    assert len(ops.mm_w8a16_dq_forward.default._schema.arguments) == 5      # ops.hpp:290-295
    assert len(ops.mlp_w8a8_quant_forward.default._schema.arguments) == 9   # ops.hpp:297-306
    assert len(ops.moe_route.default._schema.arguments) == 9
    assert len(ops.moe_permute.default._schema.arguments) == 2
    assert len(ops.moe_pack_weights.default._schema.arguments) == 6
    # the reference's own names come from the C++ extension (function-pointer registration: unnamed arguments)
    assert ops.fused_moe_fused_experts.default._schema.arguments[0].name == "_0"
    assert len(ops.enable_profile.default._schema.arguments) == 2           # ops.hpp:688-691
    assert len(ops.disable_profile.default._schema.arguments) == 0
    with pytest.raises(RuntimeError, match="closed-source"):
        ops.fused_moe_grouped_topk(*[torch.zeros(1)] * 10)
    z = torch.zeros(1, 1, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="int32"):
        ops.fused_moe_fused_experts(z, z[0], None, None, z, z, z, z, z, z, torch.zeros(1, 1, dtype=torch.int64),
                                    z[0], None, None, None, 128, 1, 1, True, 8, 4, None, None, None, False)


def test_checkpoint_layout_conversion_is_pure_data_movement(pkg, oracle):
    """convert_hf_moe_layer stacks per-expert checkpoint tensors into the packed layout; the packed
    tensors dequantise to exactly what the per-expert tensors dequantise to."""
    E, H, I = 3, 256, 128
    g = torch.Generator().manual_seed(3)
    state, pre = {}, "model.layers.3.mlp."
    for e in list(range(E)) + ["s"]:
        base = pre + ("shared_experts." if e == "s" else f"experts.{e}.")
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            q, s = oracle.quant_weight_block128(torch.randn(n, k, generator=g) * 0.05)
            state[base + proj + ".weight"], state[base + proj + ".weight_scale_inv"] = q, s
    state[pre + "gate.weight"] = torch.randn(E, H, generator=g)
    state[pre + "gate.e_score_correction_bias"] = torch.randn(E, generator=g)
    out = pkg.convert_hf_moe_layer(state, pre, E, tile_block=False)      # the last step (byte order) needs the GPU
    assert out["w13"].shape == (E, 2 * I, H) and out["w2"].shape == (E, H, I) and out["router_weight"].dtype == torch.bfloat16
    for e in range(E):
        gate = oracle.dequant_block(state[f"{pre}experts.{e}.gate_proj.weight"], state[f"{pre}experts.{e}.gate_proj.weight_scale_inv"])
        up = oracle.dequant_block(state[f"{pre}experts.{e}.up_proj.weight"], state[f"{pre}experts.{e}.up_proj.weight_scale_inv"])
        down = oracle.dequant_block(state[f"{pre}experts.{e}.down_proj.weight"], state[f"{pre}experts.{e}.down_proj.weight_scale_inv"])
        w13 = oracle.dequant_block(out["w13"][e], out["w13_scale"][e])
        assert torch.equal(w13[:I], gate) and torch.equal(w13[I:], up)
        assert torch.equal(oracle.dequant_block(out["w2"][e], out["w2_scale"][e]), down)
    sw13, sw13s, sw2, sw2s = out["shared"]
    assert sw13.shape == (1, 2 * I, H) and sw2.shape == (1, H, I) and sw13s.dtype == torch.float32
    assert torch.equal(out["bias"], state[pre + "gate.e_score_correction_bias"])


def test_size_functions_accept_an_empty_batch(pkg):
    """Workspace sizes are host arithmetic: they must not trip over a token count of zero."""
    lib = pkg._lib.lib
    assert lib.moe_permute_workspace_bytes(0, 2, 8) > 0
    assert lib.moe_fused_experts_workspace_bytes(0, 256, 128, 8, 2, 0) > 0
    assert lib.moe_fused_experts_workspace_bytes(0, 256, 128, 8, 2, 128) > 0
    assert lib.moe_layer_fp8_workspace_bytes(0, 256, 128, 8, 2, 0) > 0
    assert lib.moe_fused_experts_bf16_workspace_bytes(0, 256, 128, 8, 2) > 0
    assert lib.moe_mm_fp8_workspace_bytes(0, 256, 256) > 0
    assert lib.moe_mlp_fp8_workspace_bytes(0, 256, 128) > 0
    assert lib.moe_tile_rows(0, 2, 8) == 16


def test_derived_weight_cache_follows_the_source_tensors(pkg):
    """The drop-in ops keep packed copies of the caller's weights.  A copy must never outlive or out-date its sources:
    same tensors -> one pack; a recorded in-place change, new tensors (also on a recycled address), or an explicit
    invalidation -> a fresh pack; many layers -> every layer keeps its entry."""
    import gc
    import torch
    my_ops = pkg._my_ops
    cache = my_ops._DerivedCache()
    calls = []

    def packer(ts):
        def make():
            calls.append(1)
            return tuple(t.clone() for t in ts)
        return make

    a, b = torch.arange(8.0), torch.ones(4)
    v1 = cache.get((a, b), "x", packer((a, b)))
    v2 = cache.get((a, b), "x", packer((a, b)))
    assert v1 is v2 and len(calls) == 1
    assert cache.get((a, b), "other use", packer((a, b))) is not v1 and len(calls) == 2       # tags do not mix
    a.add_(1)                                                  # bumps the version counter
    v3 = cache.get((a, b), "x", packer((a, b)))
    assert v3 is not v1 and torch.equal(v3[0], a) and len(calls) == 3
    # an update through .data leaves no trace in the version counter: documented, cured by invalidation
    a.data.copy_(torch.zeros(8))
    assert cache.get((a, b), "x", packer((a, b))) is v3
    saved, my_ops._weights = my_ops._weights, cache
    try:
        pkg.invalidate_weight_cache()
    finally:
        my_ops._weights = saved
    v4 = cache.get((a, b), "x", packer((a, b)))
    assert v4 is not v3 and torch.equal(v4[0], torch.zeros(8))
    # freed sources take their entry with them; new tensors never meet an old copy, whatever their address
    n_before = len(cache)
    ptr = a.data_ptr()
    del a, v1, v2, v3, v4
    gc.collect()
    assert len(cache) < n_before
    for _ in range(50):
        c = torch.full((8,), 7.0)
        got = cache.get((c, b), "x", packer((c, b)))
        assert torch.equal(got[0], c)
        same_address = c.data_ptr() == ptr
        del c, got
        if same_address:
            break
    # a model with many layers, called layer after layer, twice: every layer is packed exactly once
    layers = [(torch.randn(4), torch.randn(4)) for _ in range(40)]
    calls.clear()
    for _ in range(2):
        for la in layers:
            assert torch.equal(cache.get(la, "layer", packer(la))[0], la[0])
    assert len(calls) == len(layers)


def test_ragged_weights_are_padded_to_whole_blocks_with_zero_codes(pkg):
    """H or I that 128 does not divide (the reference's weight_dequant_bc takes ceil(n/128) blocks,
    fusedMoE.pl:11-34): stacking pads gate, up and down with zero codes; every value keeps its place and its scale."""
    E, I, H = 2, 200, 320
    g = torch.Generator().manual_seed(3)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.1).to(torch.float8_e4m3fn)
    gate, up, down_t = mk(E, I, H), mk(E, I, H), mk(E, I, H)
    gs, us, ds = (torch.rand(E, 2, 3, generator=g).to(torch.bfloat16) for _ in range(3))
    w13, w13s, w2, w2s = pkg.stack_expert_weights(gate, up, down_t, gs, us, ds)
    assert tuple(w13.shape) == (E, 512, 384) and tuple(w2.shape) == (E, 384, 256)
    assert tuple(w13s.shape) == (E, 4, 3) and tuple(w2s.shape) == (E, 3, 2) and w13s.dtype == torch.float32
    b = lambda t: t.view(torch.uint8)
    assert torch.equal(b(w13)[:, :I, :H], b(gate)) and torch.equal(b(w13)[:, 256:256 + I, :H], b(up))
    assert torch.equal(b(w2)[:, :H, :I], b(down_t).transpose(1, 2))
    assert int(b(w13)[:, I:256].sum()) == 0 and int(b(w13)[:, 256 + I:].sum()) == 0 and int(b(w13)[:, :, H:].sum()) == 0
    assert int(b(w2)[:, H:].sum()) == 0 and int(b(w2)[:, :, I:].sum()) == 0
    assert torch.equal(w13s[:, :2], gs.float()) and torch.equal(w13s[:, 2:], us.float())
    assert torch.equal(w2s, ds.float().transpose(1, 2))


def test_bench_hands_on_the_offline_traffic_only_for_the_profiled_sources():
    """bench.py's roofline.traffic is an offline rocprofv3 figure kept in the profile summary: it is reported for the
    profiled workload while the kernel sources hash to the value recorded there, and withheld (None + a reason) otherwise."""
    import importlib.util
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("_bench_under_test", os.path.join(here, "..", "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    shape = (4096, 7168, 2048, 256, 8)
    got, why = bench.offline_traffic(shape)
    with open(bench.TRAFFIC_FILE) as f:
        rec = next(__import__("json").loads(l.split(None, 1)[1]) for l in f if l.startswith("TRAFFIC "))
    if rec["kernel_source_sha16"] == bench.kernel_source_hash():
        assert got == rec["bytes_per_launch"] and 7.6e9 < got < 8.2e9 and "offline" in why
    else:
        assert got is None and "stale" in why
    other, why2 = bench.offline_traffic((1, 2, 3, 4, 5))
    assert other is None and "another workload" in why2


def test_host_side_layout_arithmetic_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """The library's host-only arithmetic (workspace layout, tile heights, the bound on the tile list) built on its
    own with g++ -fsanitize=address,undefined and run here: every piece of the layout is written through, every
    bound is checked on extreme loads (tests/host_layout_check.cpp)."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = tmp_path / "host_layout_check"
    src = os.path.join(ROOT, "tests", "host_layout_check.cpp")
    r = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                        "-static-libasan", src, "-o", str(exe)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-3000:]
    r = subprocess.run([str(exe)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0 and "host layout checks passed" in r.stdout, r.stdout[-3000:]


def test_bench_refuses_more_than_one_gpu_and_its_power_roof_is_plain_arithmetic():
    """bench.py measures one GPU: `--gpus 2` exits with a message before anything touches a device.  The roof the power
    cap sets is energy over power: checked on hand numbers."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 2 and "ONE GPU" in r.stderr
    sys.path.insert(0, ROOT)
    import bench
    power = dict(read_probe=dict(watts=1100.0, ms_per_launch=1.0), first_gemm=dict(watts=1400.0, cap_watts=1400.0, ms_per_launch=1.5),
                 matrix_instructions_only=dict(watts=1300.0, tflops=4000.0), idle_watts=300.0)
    # probe: 6e12 bytes/s at 800 W above idle; matrix probe: 4 PFLOP/s at 1000 W above idle
    roof = bench.power_roof(power, nbytes=6.0e9, flops=2.0e12, probe_bytes=6.0e9)
    assert abs(roof["watts_per_tb_per_s"] - 800.0 / 6.0) < 1e-9 and abs(roof["watts_per_pflop_per_s"] - 250.0) < 1e-9
    assert abs(roof["joules_hbm"] - 0.8) < 1e-9 and abs(roof["joules_matrix"] - 0.5) < 1e-9
    assert abs(roof["floor_ms"] - 1.3 / 1100.0 * 1e3) < 1e-9
    assert bench.power_roof(dict(power, idle_watts=1500.0), 1, 1, 1) is None           # a cap below idle: no roof
    assert bench.power_roof(dict(power, read_probe=None), 1, 1, 1) is None             # counters unreadable
