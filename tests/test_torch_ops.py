"""The GEMMs as PyTorch custom operators (`torch.ops.streamk.*`): the boundary the reference reaches with
`@jit(out_idx=[2])`, which wraps its kernel as `f(A, B) -> C` (autotune/streamk_fp16_autotune.py:93-94).

CPU part: the operators are registered with the schemas the wrappers rely on, and their fake
implementations give the result's shape and dtype without touching a device.  GPU part: the operator
returns the bits of a direct C-ABI call, traces under torch.compile without a graph break, and passes
torch.library.opcheck.
"""
import ctypes

import numpy as np
import pytest


@pytest.fixture(scope="module")
def sk():
    import streamk
    return streamk


def test_operators_are_registered_with_fake_implementations(sk):
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode
    ops = torch.ops.streamk
    for name in ("gemm_f16", "gemm_bf16", "gemm_f32", "gemm_q4", "gemm_f8", "gemm_i8", "dequant_q4"):
        schema = str(getattr(ops, name).default._schema)
        assert schema.endswith("-> Tensor"), schema
        out_schema = str(getattr(ops, name + "_out").default._schema)
        assert "Tensor(a!) out" in out_schema and out_schema.endswith("-> ()"), out_schema
    with FakeTensorMode():
        h = lambda *s: torch.empty(*s, dtype=torch.float16, device="cuda")  # noqa: E731
        C = ops.gemm_f16(h(5, 64), h(32, 64))
        assert C.shape == (5, 32) and C.dtype == torch.float16 and C.device.type == "cuda" and C.stride() == (32, 1)
        assert ops.gemm_f16(h(5, 64), h(64, 32), "nn").shape == (5, 32)
        assert ops.gemm_bf16(h(5, 64).bfloat16(), h(32, 64).bfloat16()).dtype == torch.bfloat16
        assert ops.gemm_f32(h(5, 64).float(), h(64, 32).float()).shape == (5, 32)
        Wq = torch.empty(48, 128, dtype=torch.uint8, device="cuda")
        C = ops.gemm_q4(h(3, 256), Wq, h(48, 2), None)
        assert C.shape == (3, 48) and C.dtype == torch.float16
        assert ops.dequant_q4(Wq, h(48, 2), None).shape == (48, 256)
        i8 = torch.empty(7, 64, dtype=torch.int8, device="cuda")
        assert ops.gemm_i8(i8, i8).dtype == torch.int32 and ops.gemm_i8(i8, i8).shape == (7, 7)
        f8 = torch.empty(7, 64, dtype=torch.uint8, device="cuda")
        assert ops.gemm_f8(f8, f8).dtype == torch.float16
        assert ops.gemm_f16_out(h(5, 64), h(32, 64), h(5, 32)) is None


def test_configuration_strings_round_trip(sk):
    import sys
    ops = sys.modules["streamk.ops"]
    text = ops._config_string(None, dict(bm=128, schedule="basic"), dict(grid=40, fixup=None))
    assert text == "bm=128;grid=40;schedule=basic"
    assert ops._parse_config(text) == dict(bm=128, grid=40, schedule="basic")
    assert ops._config_string(None, None, {}) == ""


@pytest.mark.gpu
def test_operator_equals_direct_c_abi_call(sk):
    """torch.ops.streamk.gemm_f16(A, B) against sk_gemm_f16 called by hand with the same plan, workspace
    rules and stream: the same bits (data-parallel, and the ordered reduce)."""
    import sys
    import torch
    L = sk.lib()
    rng = np.random.default_rng(5)
    M, N, K = 300, 520, 1024
    A = torch.from_numpy((rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)).cuda()
    B = torch.from_numpy((rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)).cuda()
    for cfg in (dict(bm=128, bn=128, bk=64, schedule="dp"), dict(bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=24)):
        plan = sk.make_plan(M, N, K, "float16", "nt", cfg)
        ws = torch.zeros(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device="cuda")
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert L.sk_workspace_init(ws.data_ptr(), ws.numel(), stream) == 0
        C0 = torch.empty(M, N, dtype=torch.float16, device="cuda")
        rc = L.sk_gemm_f16(A.data_ptr(), B.data_ptr(), C0.data_ptr(), M, N, K, K, K, N, ctypes.byref(plan),
                           ws.data_ptr(), ws.numel(), stream)
        assert rc == 0
        assert L.sk_workspace_release(ws.data_ptr()) == 0
        text = sys.modules["streamk.ops"]._config_string(None, cfg, {})
        C1 = torch.ops.streamk.gemm_f16(A, B, "nt", text)
        C2 = torch.empty_like(C0)
        assert torch.ops.streamk.gemm_f16_out(A, B, C2, "nt", text) is None
        C3 = sk.streamk_fp16(A, B, **cfg)
        torch.cuda.synchronize()
        assert torch.equal(C0, C1) and torch.equal(C0, C2) and torch.equal(C0, C3), cfg
    sk.workspace_status()


@pytest.mark.gpu
def test_empty_batch_returns_an_empty_result(sk):
    """No rows of A: the operators return an empty C without a launch (torch.nn.Linear does the same); a wrong
    `out` is still refused."""
    import torch
    A = torch.empty(0, 256, dtype=torch.float16, device="cuda")
    B = torch.randn(72, 256, device="cuda").half()
    C = torch.ops.streamk.gemm_f16(A, B)
    assert C.shape == (0, 72) and C.dtype == torch.float16
    assert sk.streamk_fp16(A, B).shape == (0, 72)
    lin = sk.StreamKLinear.from_linear(torch.nn.Linear(256, 72).cuda().half())
    assert lin(A).shape == (0, 72) and lin(A.reshape(0, 3, 256)).shape == (0, 3, 72)
    out = torch.empty(0, 72, dtype=torch.float16, device="cuda")
    assert torch.ops.streamk.gemm_f16_out(A, B, out) is None
    with pytest.raises(ValueError):
        torch.ops.streamk.gemm_f16_out(A, B, torch.empty(1, 72, dtype=torch.float16, device="cuda"))


@pytest.mark.gpu
def test_linear_module_compiles_without_a_graph_break(sk):
    import torch
    import torch._dynamo
    torch.manual_seed(3)
    K, H = 1024, 1536
    layers = torch.nn.Sequential(
        sk.StreamKLinear.from_linear(torch.nn.Linear(K, H, bias=True).cuda().half(), activation="silu"),
        sk.StreamKLinear.from_linear(torch.nn.Linear(H, K, bias=True).cuda().half(), weight_format="q4"),
        sk.StreamKLinear.from_linear(torch.nn.Linear(K, H, bias=False).cuda().half(), weight_format="q4_zp"))
    x = torch.randn(2, 3, K, device="cuda").half()
    want = layers(x)
    torch._dynamo.reset()
    explained = torch._dynamo.explain(layers)(x)
    assert explained.graph_break_count == 0, explained.break_reasons
    assert explained.graph_count == 1
    compiled = torch.compile(layers, fullgraph=True, backend="aot_eager")
    got = compiled(x)
    assert got.shape == (2, 3, H) and torch.equal(got, want)
    got2 = compiled(torch.randn(5, K, device="cuda").half())   # another M: a new trace, still one graph
    assert got2.shape == (5, H)
    torch.cuda.synchronize()
    sk.workspace_status()


@pytest.mark.gpu
def test_operators_pass_opcheck(sk):
    """torch.library.opcheck: schema (the functional forms mutate nothing, the _out forms only `out`), fake
    implementation against the real one (shape, dtype, strides, device), and tracing through AOT dispatch."""
    import torch
    from torch.library import opcheck
    rng = np.random.default_rng(9)
    h = lambda *s: torch.from_numpy((rng.random(s, dtype=np.float32) * 2 - 1).astype(np.float16)).cuda()  # noqa: E731
    ops = torch.ops.streamk
    A, B = h(40, 256), h(72, 256)
    tests = ("test_schema", "test_faketensor", "test_aot_dispatch_static", "test_aot_dispatch_dynamic")
    opcheck(ops.gemm_f16.default, (A, B), test_utils=tests)
    opcheck(ops.gemm_f16.default, (A, h(256, 72), "nn", "bm=128;bn=128;schedule=basic;grid=6", h(72), "relu"), test_utils=tests)
    opcheck(ops.gemm_f16_out.default, (A, B, torch.empty(40, 72, dtype=torch.float16, device="cuda")), test_utils=tests)
    opcheck(ops.gemm_bf16.default, (A.bfloat16(), B.bfloat16()), test_utils=tests)
    opcheck(ops.gemm_f32.default, (A.float(), h(256, 72).float()), test_utils=tests)
    Wq = torch.from_numpy(rng.integers(0, 256, (72, 128), dtype=np.uint8)).cuda()
    sc = torch.from_numpy(rng.uniform(0.005, 0.02, (72, 2)).astype(np.float16)).cuda()
    opcheck(ops.gemm_q4.default, (h(4, 256), Wq, sc, None), test_utils=tests)
    opcheck(ops.gemm_q4_out.default, (h(4, 256), Wq, sc, None, torch.empty(4, 72, dtype=torch.float16, device="cuda")),
            test_utils=tests)
    opcheck(ops.dequant_q4.default, (Wq, sc, None), test_utils=tests)
    i8 = torch.from_numpy(rng.integers(-128, 128, (40, 256), dtype=np.int8)).cuda()
    opcheck(ops.gemm_i8.default, (i8, i8), test_utils=tests)
    # (raw bytes: opcheck perturbs its inputs with arithmetic torch does not have for its float8 types)
    f8a, f8b = A.to(torch.float8_e4m3fn).view(torch.uint8), B.to(torch.float8_e4m3fn).view(torch.uint8)
    opcheck(ops.gemm_f8.default, (f8a, f8b, 0.5, "e4m3"), test_utils=tests)
    torch.cuda.synchronize()
    sk.workspace_status()
