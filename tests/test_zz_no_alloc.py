"""moe_layer_fp8_static: the one-call layer entry point on the library's built-in scratch array, for callers
that cannot allocate.  Through the C ABI, on a real MI355X: its output equals moe_layer_fp8's bit for bit (the
bar for that entry point: same kernels, same order of every sum), on two calls in a row, the second on a
smaller batch (the array still holds the first call's contents), and sizes beyond the array are refused.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _call(lib, static, x, wr, bias, layer, shared, K, mode, G, TG, scale, out, logits, weights, ids, ws=None):
    T, H = x.shape
    E, I2, _ = layer[0].shape
    I_sh = shared[0].shape[1] // 2 if shared is not None else 0
    sh = [t.data_ptr() for t in shared] if shared is not None else [None] * 4
    args = [torch.cuda.current_stream().cuda_stream, x.data_ptr(), T, H, wr.data_ptr(),
            None if bias is None else bias.data_ptr(), E, K, mode, G, TG, 1, scale,
            layer[0].data_ptr(), layer[1].data_ptr(), layer[2].data_ptr(), layer[3].data_ptr(), I2 // 2,
            sh[0], sh[1], sh[2], sh[3], I_sh, out.data_ptr(), logits.data_ptr(), weights.data_ptr(), ids.data_ptr()]
    if static:
        return lib.moe_layer_fp8_static(*args)
    return lib.moe_layer_fp8(*args, ws.data_ptr(), ws.numel())


CASES = [
    # H, I, E, K, mode, groups, kept, bias, shared I, first batch, second (smaller) batch
    (1024, 256, 64, 6, 0, 1, 1, False, 0, 50, 3),             # beyond the decode size, then decode size
    (7168, 256, 256, 8, 1, 8, 4, True, 256, 32, 1),            # decode front end both times
    (512, 384, 16, 4, 1, 4, 2, True, 384, 90, 70),             # matrix-core router both times
]


@pytest.mark.parametrize("H,I,E,K,mode,G,TG,with_bias,I_sh,T1,T2", CASES)
def test_static_scratch_entry_point_equals_workspace_entry_point(pkg, oracle, dev, H, I, E, K, mode, G, TG, with_bias,
                                                                 I_sh, T1, T2):
    say("static scratch", H, I, E, K, mode, G, TG, with_bias, I_sh, T1, T2)
    lib = pkg._lib.lib
    assert lib.moe_hip_init() == 0
    layer = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=H + E)))
    shared = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(1, H, I_sh, seed=77))) if I_sh else None
    g = torch.Generator().manual_seed(E + T1)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bias = (torch.randn(E, generator=g) * 0.05).to(dev) if with_bias else None
    scale = 2.5 if mode == 1 else 1.0
    for T in (T1, T2):                                     # two calls in a row, the second smaller
        say("   T =", T)
        x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
        res = []
        for static in (False, True):
            out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=dev)
            logits = torch.empty(T, E, dtype=torch.bfloat16, device=dev)
            weights = torch.empty(T, K, dtype=torch.float32, device=dev)
            ids = torch.empty(T, K, dtype=torch.int32, device=dev)
            ws = None
            if not static:
                ws = torch.empty(pkg.layer_workspace_bytes(T, H, I, E, K, I_sh), dtype=torch.uint8, device=dev)
            rc = _call(lib, static, x, wr, bias, layer, shared, K, mode, G, TG, scale, out, logits, weights, ids, ws)
            assert rc == 0, (static, rc)
            torch.cuda.synchronize()
            res.append((out, logits, weights, ids))
        (o0, l0, w0, i0), (o1, l1, w1, i1) = res
        assert torch.isfinite(o0.float()).all()
        assert torch.equal(i0, i1) and torch.equal(w0, w1)
        assert torch.equal(l0.view(torch.int16), l1.view(torch.int16))
        assert torch.equal(o0.view(torch.int16), o1.view(torch.int16))
        # the Python wrapper takes the same road
        o2 = pkg.layer_fp8(x, wr, *layer, K, "sigmoid" if mode else "softmax", bias=bias, n_groups=G, topk_groups=TG,
                           renorm=True, scale=scale, shared=shared, static_scratch=True)
        torch.cuda.synchronize()
        assert torch.equal(o2.view(torch.int16), o0.view(torch.int16))


def _hip_runtime():
    """The HIP runtime this process already runs on (the very library torch and libmoe_hip.so are bound to)."""
    import ctypes
    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64.so" in line})
    assert paths, "no HIP runtime is mapped into this process"
    hip = ctypes.CDLL(paths[0])
    hip.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    hip.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    return hip


def test_static_scratch_entry_point_allocates_nothing_and_works_in_the_library_array(pkg, oracle, dev):
    """What the entry point exists for: with inputs and outputs in place the call allocates nothing - neither through
    torch's allocator nor from the device directly - and its kernels work inside the array whose address
    hipGetSymbolAddress gave (moe_static_scratch_address): the array is poisoned, the call runs, the poison is gone
    from the array's front (where the workspace layout starts) and the result is right."""
    import ctypes
    say("static scratch: no allocation, scratch inside the library's array")
    lib = pkg._lib.lib
    hip = _hip_runtime()
    H, I, E, K, T = 1024, 256, 64, 6, 40
    layer = pkg.pack_layer(*(t.to(dev) for t in oracle.make_layer(E, H, I, seed=5)))
    g = torch.Generator().manual_seed(9)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    outs = [torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    logits = torch.empty(T, E, dtype=torch.bfloat16, device=dev)
    weights = torch.empty(T, K, dtype=torch.float32, device=dev)
    ids = torch.empty(T, K, dtype=torch.int32, device=dev)
    ws = torch.empty(pkg.layer_workspace_bytes(T, H, I, E, K, 0), dtype=torch.uint8, device=dev)
    assert lib.moe_hip_init() == 0
    addr = ctypes.c_void_p()
    assert lib.moe_static_scratch_address(ctypes.byref(addr)) == 0 and addr.value and addr.value % 256 == 0
    again = ctypes.c_void_p()
    assert lib.moe_static_scratch_address(ctypes.byref(again)) == 0 and again.value == addr.value
    n = 16 << 20
    # the array is no part of any torch allocation made here
    for t in (x, wr, ws, *outs, *layer):
        lo = t.data_ptr()
        assert addr.value + n <= lo or lo + t.numel() * t.element_size() <= addr.value
    assert _call(lib, False, x, wr, None, layer, None, K, 0, 1, 1, 1.0, outs[0], logits, weights, ids, ws) == 0
    torch.cuda.synchronize()
    assert hip.hipMemset(addr, 0xA5, n) == 0
    torch.cuda.synchronize()
    free0, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free0), ctypes.byref(total)) == 0
    stats0 = torch.cuda.memory_stats()
    mem0 = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), stats0["allocation.all.allocated"],
            stats0["segment.all.allocated"])
    rc = _call(lib, True, x, wr, None, layer, None, K, 0, 1, 1, 1.0, outs[1], logits, weights, ids)
    torch.cuda.synchronize()
    stats1 = torch.cuda.memory_stats()
    mem1 = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), stats1["allocation.all.allocated"],
            stats1["segment.all.allocated"])
    free1 = ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free1), ctypes.byref(total)) == 0
    assert rc == 0
    assert mem1 == mem0, "the call went through torch's allocator"
    assert free1.value == free0.value, "the call changed the device's free memory"
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    host = (ctypes.c_ubyte * n)()
    assert hip.hipMemcpy(host, addr, n, 2) == 0                  # 2 = device to host
    raw = ctypes.string_at(host, n)
    assert raw[:4096] != b"\xa5" * 4096, "the kernels did not write into the library's array"
    need = pkg.layer_workspace_bytes(T, H, I, E, K, 0)
    assert raw[need + 256:] == b"\xa5" * (n - need - 256), "a kernel wrote past the problem's share of the array"


def test_static_scratch_entry_point_refuses_what_does_not_fit(pkg, dev):
    say("static scratch limits")
    lib = pkg._lib.lib
    # the DeepSeek-V3 layer at T=4096 needs hundreds of MB: refused on the sizes alone, nothing is launched and
    # no pointer is touched
    assert pkg.layer_workspace_bytes(4096, 7168, 2048, 256, 8, 2048) > (16 << 20)
    rc = lib.moe_layer_fp8_static(None, 1, 4096, 7168, 1, None, 256, 8, 1, 8, 4, 1, 2.5, 1, 1, 1, 1, 2048, 1, 1, 1, 1,
                                  2048, 1, None, None, None)
    assert rc == -6
    assert b"scratch" in lib.moe_hip_strerror(rc)
    assert lib.moe_layer_fp8_static(None, 1, 1, 7168, 1, None, 1300, 8, 1, 8, 4, 1, 2.5, 1, 1, 1, 1, 2048, None, None,
                                    None, None, 0, 1, None, None, None) == -2          # more than 1024 experts
