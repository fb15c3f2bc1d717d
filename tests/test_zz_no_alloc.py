"""sk_gemm_f16_static: the entry point that allocates nothing (its fix-up workspace is an array inside the
library's code object) must return what sk_gemm_f16 returns with a caller's workspace -- bit for bit with the
ordered reduce, and with the atomic fix-up on integer data, whose sums are exact in any order.  Called twice in
a row, the second time on a smaller problem, so that the second call meets the first one's leftovers."""
import ctypes

import numpy as np
import pytest


@pytest.mark.gpu
def test_static_workspace_entry_point_matches_sk_gemm_f16():
    import torch
    import streamk
    L = streamk.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(2024)

    def both(M, N, K, cfg, integer):
        if integer:
            A = rng.integers(-1, 2, (M, K)).astype(np.float16)
            B = rng.integers(-1, 2, (N, K)).astype(np.float16)
        else:
            A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
            B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        plan = streamk.make_plan(M, N, K, "float16", "nt", cfg)
        assert plan.streamk_tiles > 0 and 0 < plan.workspace_bytes <= 64 * 1024 * 1024 + 262144 + 256, cfg
        ws = torch.empty(int(plan.workspace_bytes), dtype=torch.uint8, device="cuda")
        assert L.sk_workspace_init(ws.data_ptr(), ws.numel(), stream) == 0
        want = torch.empty(M, N, dtype=torch.float16, device="cuda")
        assert L.sk_gemm_f16(dA.data_ptr(), dB.data_ptr(), want.data_ptr(), M, N, K, K, K, N, ctypes.byref(plan),
                             ws.data_ptr(), ws.numel(), stream) == 0
        got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        print(f"static call {M}x{N}x{K} {cfg}", flush=True)
        assert L.sk_gemm_f16_static(dA.data_ptr(), dB.data_ptr(), got.data_ptr(), M, N, K, K, K, N, ctypes.byref(plan),
                                    stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert L.sk_workspace_release(ws.data_ptr()) == 0
        assert torch.equal(got, want), (M, N, K, cfg)
        if integer:
            assert np.array_equal(got.cpu().numpy().astype(np.int32), A.astype(np.int32) @ B.astype(np.int32).T)

    red = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=64)
    atm = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="atomic", grid=64)
    # two calls in a row, the second on a smaller problem: ordered reduce (random data, bit-reproducible) ...
    both(1000, 1096, 4104, red, integer=False)
    both(520, 264, 1032, dict(red, grid=24), integer=False)
    # ... then the atomic fix-up on what the reduce calls left behind, again large then small (exact integer data)
    both(1000, 1096, 4104, atm, integer=True)
    both(520, 264, 1032, dict(atm, grid=24), integer=True)
    both(520, 264, 1032, dict(red, grid=24), integer=True)
    # the large tile of the headline kernel
    both(1024, 1024, 2048, dict(bm=256, bn=256, bk=64, schedule="basic", fixup="reduce", grid=48), integer=False)
    # tiles cut into four equal segments: the two-round exchange and its second set of flags
    both(512, 512, 1024, dict(bm=128, bn=128, bk=64, schedule="splitk", split=4, fixup="reduce"), integer=False)
    both(512, 512, 1024, dict(bm=256, bn=256, bk=64, schedule="splitk", split=4, fixup="reduce"), integer=True)
    # a plan without Stream-K tiles needs no workspace at all
    plan = streamk.make_plan(512, 512, 512, "float16", "nt", dict(bm=128, bn=128, bk=64, schedule="dp"))
    A = torch.randn(512, 512, device="cuda").half()
    C = torch.empty(512, 512, dtype=torch.float16, device="cuda")
    assert L.sk_gemm_f16_static(A.data_ptr(), A.data_ptr(), C.data_ptr(), 512, 512, 512, 512, 512, 512,
                                ctypes.byref(plan), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(C, streamk.streamk_fp16(A, A, bm=128, bn=128, bk=64, schedule="dp"))
    # a plan that needs more than the static array holds is refused
    big = streamk.make_plan(8192, 8192, 8192, "float16", "nt", dict(bm=256, bn=256, bk=64, schedule="basic", fixup="atomic", grid=255))
    assert big.workspace_bytes > 64 * 1024 * 1024 + 262144 + 256
    assert L.sk_gemm_f16_static(A.data_ptr(), A.data_ptr(), C.data_ptr(), 8192, 8192, 8192, 8192, 8192, 8192,
                                ctypes.byref(big), stream) == -5


@pytest.mark.gpu
def test_static_entry_point_replays_from_a_hip_graph():
    """sk_gemm_f16_static recorded into a HIP graph (after sk_static_init, so that the capture holds kernel launches
    only) must give on every replay what the eager call gives, bit for bit: ordered reduce on random data, atomic
    fix-up on integer data.  Between the replays the program runs eager calls of the other fix-up on the same
    static array and synchronises, so that each replay meets different leftovers."""
    import torch
    import streamk
    L = streamk.lib()
    assert L.sk_static_init() == 0
    rng = np.random.default_rng(77)
    M, N, K = 520, 776, 2056
    red = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=40)
    atm = dict(red, fixup="atomic")

    def operands(integer):
        if integer:
            A = rng.integers(-1, 2, (M, K)).astype(np.float16)
            B = rng.integers(-1, 2, (N, K)).astype(np.float16)
        else:
            A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
            B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        return torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()

    def call(dA, dB, out, plan, stream):
        return L.sk_gemm_f16_static(dA.data_ptr(), dB.data_ptr(), out.data_ptr(), M, N, K, K, K, N,
                                    ctypes.byref(plan), ctypes.c_void_p(stream.cuda_stream))

    for cfg, other, integer in ((red, atm, False), (atm, red, True)):
        dA, dB = operands(integer)
        plan = streamk.make_plan(M, N, K, "float16", "nt", cfg)
        other_plan = streamk.make_plan(M, N, K, "float16", "nt", other)
        assert plan.streamk_tiles > 0 and other_plan.streamk_tiles > 0
        want = torch.empty(M, N, dtype=torch.float16, device="cuda")
        assert call(dA, dB, want, plan, torch.cuda.current_stream()) == 0
        torch.cuda.synchronize()
        got = torch.empty(M, N, dtype=torch.float16, device="cuda")
        scratch_out = torch.empty(M, N, dtype=torch.float16, device="cuda")
        graph = torch.cuda.CUDAGraph()
        print(f"capture {cfg['fixup']}", flush=True)
        with torch.cuda.graph(graph):
            assert call(dA, dB, got, plan, torch.cuda.current_stream()) == 0
        for replay in range(3):
            got.fill_(float("nan"))
            print(f"replay {replay} {cfg['fixup']}", flush=True)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(got, want), (cfg["fixup"], replay)
            assert call(dA, dB, scratch_out, other_plan, torch.cuda.current_stream()) == 0
            torch.cuda.synchronize()
        if integer:
            ref = dA.cpu().numpy().astype(np.int32) @ dB.cpu().numpy().astype(np.int32).T
            assert np.array_equal(got.cpu().numpy().astype(np.int32), ref)
