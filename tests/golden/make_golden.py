"""Writes the small fixtures under tests/golden/ from the CPU oracle.

The reference ships no golden files (its scripts assert against a dense matmul at run time), so the
vectors are produced by this repository's own restatement of the reference arithmetic; the oracle is
pinned independently in tests/test_oracle_*.py.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as o  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.default_rng(0)
    # ragged Stream-K case: 48x40x72, 16x8x8 tiles on 7 simulated CTAs (15 tiles, 9 iters each, 8 of them split)
    A = (rng.random((48, 72), dtype=np.float32) * 2 - 1)
    B = (rng.random((72, 40), dtype=np.float32) * 2 - 1)
    part = o.partition(48, 40, 72, 16, 8, 8, 7)
    np.savez(os.path.join(OUT, "streamk_f32_48x40x72.npz"), A=A, B=B,
             C_atomic=o.streamk_gemm_f32(A, B, 16, 8, 8, 7, fixup="atomic"),
             C_reduce=o.streamk_gemm_f32(A, B, 16, 8, 8, 7, fixup="reduce"),
             partition=np.array([part[k] for k in sorted(part)], dtype=np.int32),
             partition_keys=np.array(sorted(part)))
    # fp16 NT case with edges in M, N and K for the GPU kernels (expected C in fp32)
    A16 = (rng.random((200, 328), dtype=np.float32) * 2 - 1).astype(np.float16)
    B16 = (rng.random((136, 328), dtype=np.float32) * 2 - 1).astype(np.float16)
    np.savez(os.path.join(OUT, "gemm_f16_nt_200x136x328.npz"), A=A16, B=B16,
             C=o.matmul_fp32(A16, B16, trans_b=True))
    # Q4: every nibble value in every position of a 32-bit word, two scale groups per row
    N, K = 16, 256
    q = np.empty((N, K), dtype=np.uint8)
    for n in range(N):
        for k in range(K):
            q[n, k] = (n + 3 * k + (k // 8)) % 16
    Wq = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    scales = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    Aq = rng.standard_normal((4, K)).astype(np.float16)
    np.savez(os.path.join(OUT, "q4_16x256.npz"), Wq=Wq, scales=scales, nibbles=q,
             W=o.dequant_q4(Wq, scales, 128, 8), A=Aq, C=o.q4_gemm_ref(Aq, Wq, scales, 128, 8))
    print("fixtures written to", OUT)


if __name__ == "__main__":
    main()
