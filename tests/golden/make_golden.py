"""Writes the fixtures under tests/golden/.

genmat_seed7_4096.npy   first 4096 values of the reference's genMat stream (utils.h:25-33),
                        produced by the reference's own header compiled into
                        oracle/_ref/librefutils.so -- run in the container that has the
                        reference checkout.
small_case.npz          a 48 x 208 x 384 problem: inputs in the kernel layouts and the
                        oracle's bf16 result (regression pin of the oracle across rebuilds
                        and compilers; the reference holds no vectors for this path).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    ref = oracle.refutils()
    if ref is not None:
        out = np.empty(4096, np.float32)
        ref.ref_genMat(out.ctypes.data, out.size)
        np.save(os.path.join(HERE, "genmat_seed7_4096.npy"), out)
    m, n, k = 48, 208, 384
    a, b, sa, sb = oracle.make_inputs(m, n, k, 4242, 1.0, 50.0)
    c = oracle.ref_gemm_naive(a, b, sa, sb, m, n, k)
    np.savez_compressed(os.path.join(HERE, "small_case.npz"), a=a, b=b, a_scale=sa, b_scale=sb, c=c,
                        shape=np.array([m, n, k]))


if __name__ == "__main__":
    main()
