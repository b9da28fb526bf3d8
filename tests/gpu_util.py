"""Helpers for the GPU parity tests: run one case through the C ABI and check it against the oracle."""
import numpy as np
import torch

from onnxruntime_amd.matmul_nbits import MatMulNBits

FP32_GATE = 1e-4   # max |err| <= 1e-4 * sum_k |a_k w_kn|   (fp32 models)
FP16_GATE = 5e-3   # relative L2 error                      (fp16 models)


def tdtype(np_dtype):
    return torch.float16 if np.dtype(np_dtype) == np.float16 else torch.float32


def dev(x):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()


def make_op(case, prepack=True):
    op = MatMulNBits(case.K, case.N, case.bits, case.block_size, dtype=tdtype(case.dtype),
                     has_zero_points=case.zero_points is not None, has_bias=case.bias is not None)
    if prepack:
        assert op.PrePack(dev(case.B), dev(case.scales), dev(case.zero_points))
    return op


def run_case(case, prepack=True, A=None):
    op = make_op(case, prepack)
    a = dev(case.A if A is None else A)
    if prepack:
        y = op.Compute(a, bias=dev(case.bias))
    else:
        y = op.Compute(a, dev(case.B), dev(case.scales), dev(case.zero_points), dev(case.bias))
    torch.cuda.synchronize()
    return y.cpu().numpy()


def check_against_oracle(oracle, case, y, A=None, nthreads=8):
    A = case.A if A is None else A
    y64, bound = oracle.C.matmul_f64(A, case.B, case.scales, case.zero_points, case.bias, case.N, case.K, case.bits,
                                     case.block_size, nthreads=nthreads)
    err = np.abs(y.astype(np.float64) - y64)
    if np.dtype(case.dtype) == np.float32:
        worst = float(np.max(err / (bound + 1e-30)))
        assert worst <= FP32_GATE, f"max |err| / row bound = {worst:.3e} > {FP32_GATE}"
        return worst
    rel = float(np.linalg.norm(err) / max(np.linalg.norm(y64), 1e-30))
    assert rel <= FP16_GATE, f"relative L2 = {rel:.3e} > {FP16_GATE}"
    # and against the reference-semantics result itself (fp32 accumulate, one narrowing): a few half ulps at most
    yref = oracle.C.matmul(A, case.B, case.scales, case.zero_points, case.bias, case.N, case.K, case.bits,
                           case.block_size, nthreads=nthreads).astype(np.float64)
    rel_ref = float(np.linalg.norm(y.astype(np.float64) - yref) / max(np.linalg.norm(yref), 1e-30))
    assert rel_ref <= FP16_GATE
    return rel
