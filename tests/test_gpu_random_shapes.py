"""GPU parity on seeded random draws of shape, operand type, plan and epilogue: what a caller gets who does not
pick from the shapes the other tests name.  Every case goes through the C ABI and is checked against the CPU
oracle's fp32 host product of the same inputs (max|C - ref| / max|ref|; the reference asserts rtol = atol = 1e-2,
streamk_fp32.py:208; fp16 results here stay within 2e-3, bfloat16 within 1e-2, Q4 within 2e-3 of the product
with the dequantised weights).  Padded rows of C must keep the NaNs they were filled with.
"""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 4, 5, 8, 9, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 200]
COLS = [16, 48, 100, 250, 512, 1000, 1024, 2048, 2050, 4096, 5120, 8192, 11008]
DEPTHS = [256, 512, 768, 1024, 1280, 2048, 4096, 4352, 5120, 8192]
# tiles of the kernels that stream fp16 / bfloat16 weights through LDS (up to 96 rows of A)
STREAM_TILES = [(16, 16, 1024), (16, 32, 512), (16, 64, 256), (32, 32, 256), (32, 64, 256), (64, 32, 256), (64, 64, 256),
                (96, 32, 256)]


@pytest.fixture(scope="module")
def sk():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import streamk
    streamk.lib()
    assert "libstreamk.so" in open("/proc/self/maps").read(), "native library not loaded"
    return streamk


def _draw_config(rnd, M):
    """An explicit plan on one of the streaming kernels: any schedule and fix-up the planner may be asked for."""
    tiles = [t for t in STREAM_TILES if t[0] >= M and not (t[0] >= 2 * M and t[0] > 16)]
    bm, bn, bk = rnd.choice(tiles)
    sched = rnd.choice(["dp", "dp", "sk1", "sk2", "basic", "splitk"])
    cfg = dict(bm=bm, bn=bn, bk=bk, variant=5, schedule=sched)
    if sched == "splitk":
        cfg.update(fixup=rnd.choice(["reduce", "atomic"]), split=rnd.choice([2, 3, 4]))
    elif sched != "dp":
        cfg.update(fixup=rnd.choice(["reduce", "atomic"]), grid=rnd.choice([64, 100, 256]))
    elif rnd.random() < 0.3:
        cfg["grid"] = rnd.choice([5, 64, 256])
    return cfg


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_16_bit_shapes_plans_and_epilogues(sk, oracle, seed):
    import torch
    rnd = random.Random(seed)
    rng = np.random.default_rng(seed)
    ran, kernels = 0, set()
    for it in range(120):
        M, N, K = rnd.choice(ROWS), rnd.choice(COLS), rnd.choice(DEPTHS)
        name = rnd.choice(["float16", "bfloat16"])
        tdt, run, tol = (torch.float16, sk.streamk_fp16, 2e-3) if name == "float16" else (torch.bfloat16, sk.streamk_bf16, 1e-2)
        pad_a, pad_c = rnd.choice([0, 0, 8, 64]), rnd.choice([0, 0, 8, 24])
        abuf = torch.from_numpy(rng.standard_normal((M, K + pad_a), dtype=np.float32) * 0.5).to(tdt).cuda()
        A = abuf[:, :K]
        W = torch.from_numpy(rng.standard_normal((N, K), dtype=np.float32) * 0.05).to(tdt).cuda()
        cbuf = torch.full((M, N + pad_c), float("nan"), dtype=tdt, device="cuda")
        C = cbuf[:, :N]
        bias = torch.from_numpy(rng.standard_normal(N, dtype=np.float32)).to(tdt).cuda() if rnd.random() < 0.4 else None
        act = rnd.choice([None, None, "relu", "silu", "gelu_tanh"])
        cfg = _draw_config(rnd, M) if M <= 96 and rnd.random() < 0.6 else None
        case = (seed, it, name, M, N, K, pad_a, pad_c, bias is not None, act, cfg)
        try:
            plan = sk.make_plan(M, N, K, name, "nt", cfg) if cfg else sk.make_plan(M, N, K, name, "nt", use_tuned=rnd.random() < 0.5)
        except sk.StreamKError:
            assert cfg is not None, case  # only an explicit configuration may be turned down (e.g. a split K does not divide into)
            continue
        run(A, W, out=C, plan=plan, bias=bias, activation=act)
        ref = oracle.matmul_fp32(A.float().cpu().numpy(), W.float().cpu().numpy(), trans_b=True)
        if bias is not None:
            ref = ref + bias.float().cpu().numpy()
        ref = oracle.activation_ref(ref, act)
        scale = max(float(np.max(np.abs(ref))), 1.0)
        err = float(np.max(np.abs(C.double().cpu().numpy() - ref)))
        assert err <= tol * scale + 1e-3, (case, sk.kernel_name(plan.kernel_id), plan.grid, err)
        assert pad_c == 0 or bool(torch.isnan(cbuf[:, N:].float()).all()), (case, "wrote past the row end")
        kernels.add(sk.kernel_name(plan.kernel_id))
        ran += 1
    assert ran >= 100 and len(kernels) >= 8, (ran, sorted(kernels))


def test_random_q4_shapes(sk, oracle):
    import torch
    rnd = random.Random(5)
    rng = np.random.default_rng(5)
    kernels = set()
    for it in range(60):
        M, N = rnd.choice(ROWS), rnd.choice(COLS)
        K = rnd.choice([128, 256, 512, 1024, 1280, 2048, 4096, 4352, 8192])
        A = (rng.standard_normal((M, K), dtype=np.float32) * 0.5).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        plan = sk.make_plan(M, N, K, "q4", "nt", use_tuned=rnd.random() < 0.5)
        C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        sk.streamk_q4(torch.from_numpy(A).cuda(), torch.from_numpy(Wq).cuda(), torch.from_numpy(sc).cuda(), out=C, plan=plan)
        ref = oracle.q4_gemm_ref(A, Wq, sc, 128, 8)
        err = oracle.max_abs_rel(C.float().cpu().numpy(), ref)
        assert err <= 2e-3, (it, M, N, K, sk.kernel_name(plan.kernel_id), plan.grid, err)
        kernels.add(sk.kernel_name(plan.kernel_id))
    assert len(kernels) >= 5, sorted(kernels)
