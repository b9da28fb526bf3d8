"""fp32 models with few rows (from 5, up to where the tile GEMM's grid fills the chip): the kernel that feeds packed weights from registers to the fp32 matrix cores
(mnb_rows16_f32.hip), through the C ABI, against the CPU oracle (reference semantics, fp32 tolerance
|err| <= 1e-4 * sum|a * w|) and bit-exactly on unit-vector rows (the weights are dequantised as (q - zp) * scale, the
reference's fp32 dequantisation)."""
import numpy as np
import pytest

from gpu_util import check_against_oracle, run_case
from onnxruntime_amd import _lib
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu
KERNEL = "mnb_rows16_f32_kernel"


def kernel_name(M, N, K, bits, bs):
    return _lib.load().MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT).decode()


# N selects the column tiles per workgroup (one, two, four), K the wavefronts per workgroup (4, 8, 16) and whether the
# last chunk of four k-groups is partly empty
SHAPES = [(5, 70, 96), (16, 300, 512), (17, 1000, 1024), (33, 4096, 2048), (64, 520, 4096), (48, 7200, 1056),
          (9, 14336, 4096), (64, 14336, 512), (40, 3600, 8192), (12, 64, 160), (300, 1000, 512), (130, 4096, 1024)]


@pytest.mark.parametrize("bits,bs,zp,bias", [(4, 32, True, True), (4, 128, False, False), (4, 16, True, False),
                                             (4, 16, False, True), (8, 64, True, True), (8, 16, False, False),
                                             (8, 256, True, False), (2, 32, True, True)])
def test_parity(oracle, bits, bs, zp, bias):
    for (M, N, K) in SHAPES:
        assert kernel_name(M, N, K, bits, bs) == KERNEL, (M, N, K)
        c = make_case(M, N, K, bits, bs, np.float32, has_zp=zp, has_bias=bias, seed=M + N + K)
        check_against_oracle(oracle, c, run_case(c))


@pytest.mark.parametrize("bits,bs,N,K", [(4, 32, 70, 96), (4, 16, 300, 512), (8, 64, 130, 256), (4, 128, 1100, 4096),
                                         (8, 16, 2300, 1040), (2, 64, 90, 1024)])
def test_unit_rows_recover_the_dequantised_weights(oracle, bits, bs, N, K):
    """Rows that are unit vectors e_k push column k of W through the kernel unchanged: bit for bit the reference's
    fp32 dequantisation, whatever the scales."""
    for M in (5, 16, 64):
        assert kernel_name(M, N, K, bits, bs) == KERNEL
        c = make_case(M, N, K, bits, bs, np.float32, has_zp=True, seed=3)
        ks = np.random.default_rng(M).choice(K, size=M, replace=False)
        a = np.zeros((M, K), np.float32)
        a[np.arange(M), ks] = 1.0
        want = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs)[:, ks].T
        y = run_case(c, A=a)
        assert np.array_equal(y.view(np.uint32), np.ascontiguousarray(want, np.float32).view(np.uint32))


def test_rows_and_k_outside_its_range_take_the_other_kernels():
    assert kernel_name(4, 4096, 4096, 4, 32) == "mnb_gemv_kernel"
    assert kernel_name(512, 4096, 4096, 4, 32) == KERNEL             # the tile GEMM's grid would be one round
    assert kernel_name(2048, 4096, 4096, 4, 32) == "mnb_gemm32_kernel"
    assert kernel_name(16, 4096, 4100, 4, 32) != KERNEL   # K is not a whole number of k-groups
