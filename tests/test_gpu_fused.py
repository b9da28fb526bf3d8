"""GPU parity of the fused projections (MatMulNBitsMlp / MatMulNBitsQkv and their normalisation prologue), called
through the C ABI, against the CPU oracle.

Gates: fp16 models relative L2 <= 5e-3 against the fp64 evaluation and a few half ulps against the oracle's
reference-semantics result; fp32 models max |err| <= 1e-4 * (first-order bound from sum_k |a w| of both projections).
"""
import numpy as np
import pytest
import torch

from gpu_util import FP16_GATE, FP32_GATE, dev, tdtype
from onnxruntime_amd import _lib
from onnxruntime_amd.matmul_nbits import MatMulNBitsMlp, MatMulNBitsQkv, simplified_layer_norm
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu


def _ulps(got, want):
    g, w = got.astype(np.float32), want.astype(np.float32)
    sp = np.spacing(np.maximum(np.abs(want), np.finfo(want.dtype).tiny)).astype(np.float32)
    return np.abs(g - w) / sp


def _mats(M, N, K, bits, bs, dtype, bias, seed):
    c = make_case(M, N, K, bits, bs, dtype, has_bias=bias, seed=seed)
    return c, (c.B, c.scales, c.bias)


def _norm_inputs(M, K, dtype, skip_rows, seed):
    rng = np.random.default_rng(seed)
    gamma = rng.uniform(0.5, 1.5, K).astype(dtype)
    skip = None if skip_rows == 0 else rng.standard_normal((skip_rows, K)).astype(dtype)
    return skip, gamma


# ------------------------------------------------------------------------------------------------ normalisation
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("M,K,skip_rows", [(1, 4096, 1), (3, 4096, 0), (5, 96, 5), (4, 100, 2), (2, 14336, 2),
                                            (1, 40000, 1), (7, 8200, 0)])
def test_simplified_layer_norm(oracle, dtype, M, K, skip_rows):
    rng = np.random.default_rng(M * K)
    x = rng.standard_normal((M, K)).astype(dtype)
    skip, gamma = _norm_inputs(M, K, dtype, skip_rows, 5)
    eps = 1e-5
    if skip is None:
        got = simplified_layer_norm(dev(x), dev(gamma), eps).cpu().numpy()
        want = oracle.C.simplified_layer_norm(x, None, gamma, eps)
    else:
        got, got_sum = simplified_layer_norm(dev(x), dev(gamma), eps, skip=dev(skip), want_skip_sum=True)
        got, got_sum = got.cpu().numpy(), got_sum.cpu().numpy()
        want, want_sum = oracle.C.simplified_layer_norm(x, skip, gamma, eps, want_sum=True)
        assert np.array_equal(got_sum, want_sum)  # one exact fp32 addition, one narrowing
    # the sum of squares is accumulated in another order (a tree; the reference's loop is sequential in fp32)
    u = _ulps(got, want)
    if dtype == np.float16:
        assert u.max() <= 1 and (u == 0).mean() >= 0.99, (u.max(), (u == 0).mean())
    else:
        s64 = x.astype(np.float64) + (0 if skip is None else np.resize(skip.astype(np.float64), x.shape))
        ref = (s64 / np.sqrt((s64 ** 2).mean(-1, keepdims=True) + eps) * gamma.astype(np.float64))
        assert _ulps(got, ref.astype(np.float32)).max() <= 4       # against the exact value
        assert u.max() <= 2e-7 * np.sqrt(K) / 2 ** -23 + 4, u.max()  # the sequential sum's own error grows with K


# ------------------------------------------------------------------------------------------------ MLP
def _check_mlp(oracle, got, A_act, g, u, N, K, bits, bs, dtype):
    gm, um = (g.B, g.scales, g.bias), (u.B, u.scales, u.bias)
    g64, gb = oracle.C.matmul_f64(A_act, g.B, g.scales, None, g.bias, N, K, bits, bs, nthreads=8)
    u64, ub = oracle.C.matmul_f64(A_act, u.B, u.scales, None, u.bias, N, K, bits, bs, nthreads=8)
    sig = 1.0 / (1.0 + np.exp(-g64))
    ref = g64 * sig * u64
    err = np.abs(got.astype(np.float64) - ref)
    # d(silu)/dg <= 1.1: first-order propagation of the two products' own bounds sum_k |a w|
    bound = 1.1 * np.abs(u64) * gb + np.abs(g64 * sig) * ub
    if dtype == np.float32:
        worst = float(np.max(err / (bound + 1e-30)))
        assert worst <= FP32_GATE, worst
    else:
        rel = float(np.linalg.norm(err) / max(np.linalg.norm(ref), 1e-30))
        assert rel <= FP16_GATE, rel
        # element by element: the kernels may round each dequantised weight to fp16 (2^-11 relative, as the
        # reference's fp16 dequantisation does) and narrow the result once
        assert np.all(err <= 1e-3 * bound + 2.0 ** -10 * np.abs(ref) + 1e-7), float(np.max(err / (bound + 1e-30)))
        want = oracle.C.mlp(A_act, gm, um, N, K, bits, bs, nthreads=8).astype(np.float64)
        assert float(np.linalg.norm(got.astype(np.float64) - want) / max(np.linalg.norm(want), 1e-30)) <= FP16_GATE


MLP_CASES = [
    # M, N, K, bits, bs: decode kernel (aligned / ragged K), streaming kernel, tile GEMM, odd widths
    (1, 64, 128, 4, 32), (1, 1000, 512, 4, 128), (4, 40, 96, 4, 16), (16, 333, 256, 8, 64), (2, 48, 100, 4, 32),
    (17, 100, 256, 4, 32), (64, 512, 512, 4, 128), (100, 72, 320, 8, 32), (300, 520, 256, 4, 64),
    (512, 1024, 1024, 4, 32), (2048, 2048, 1024, 4, 32), (2048, 2040, 1024, 4, 128), (2048, 2044, 1024, 4, 32),
]


def test_mlp_cases_cover_every_kernel():
    lib = _lib.load()
    names = {lib.MnbGemmKernelName(M, 2 * ((N + 15) // 16 * 16), K, bits, bs, _lib.DTYPE_FLOAT16).decode()
             for (M, N, K, bits, bs) in MLP_CASES}
    assert {"mnb_skinny_kernel", "mnb_mid_kernel", "mnb_gemm256_kernel"} <= names, names


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("M,N,K,bits,bs", MLP_CASES)
def test_mlp_parity(oracle, dtype, bias, M, N, K, bits, bs):
    g, gm = _mats(M, N, K, bits, bs, dtype, bias, 11)
    u, um = _mats(M, N, K, bits, bs, dtype, bias and N % 2 == 0, 12)  # sometimes only one of the two biases
    op = MatMulNBitsMlp(K, N, bits, bs, dtype=tdtype(dtype))
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), dev(u.bias))
    y = op.Compute(dev(g.A))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (M, N)
    _check_mlp(oracle, y.cpu().numpy(), g.A, g, u, N, K, bits, bs, dtype)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("M,N,K,skip_rows,want_sum", [(1, 512, 1024, 1, True), (3, 100, 256, 0, False),
                                                       (8, 96, 200, 8, True), (40, 256, 512, 1, False),
                                                       (300, 512, 256, 300, True)])
def test_mlp_with_norm_prologue(oracle, dtype, M, N, K, skip_rows, want_sum):
    bits, bs = 4, 32
    g, gm = _mats(M, N, K, bits, bs, dtype, True, 21)
    u, um = _mats(M, N, K, bits, bs, dtype, False, 22)
    skip, gamma = _norm_inputs(M, K, dtype, skip_rows, 23)
    op = MatMulNBitsMlp(K, N, bits, bs, epsilon=1e-5, dtype=tdtype(dtype))
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), None)
    a3 = g.A.reshape(1, M, K)  # leading dimensions are kept
    out = op.Compute(dev(a3), skip=dev(skip), norm_scale=dev(gamma), want_skip_sum=want_sum)
    torch.cuda.synchronize()
    y = (out[0] if want_sum else out).cpu().numpy()
    assert y.shape == (1, M, N)
    if skip is None:
        act = oracle.C.simplified_layer_norm(g.A, None, gamma, 1e-5)
    else:
        act, sm = oracle.C.simplified_layer_norm(g.A, skip, gamma, 1e-5, want_sum=True)
        if want_sum:
            assert np.array_equal(out[1].cpu().numpy().reshape(M, K), sm)
    # the device's normalised activation may differ from the oracle's by one rounding in a few places: the products
    # are checked against the device's own normalisation, which the test above holds to the oracle
    act_dev = simplified_layer_norm(dev(g.A), dev(gamma), 1e-5, skip=dev(skip)).cpu().numpy()
    assert _ulps(act_dev, act).max() <= (1 if dtype == np.float16 else 64)
    _check_mlp(oracle, y.reshape(M, N), act_dev, g, u, N, K, bits, bs, dtype)


def test_mlp_equals_two_gemms_and_silu(oracle):
    """The fused call against the product's own unfused route (two MatMulNBits + elementwise), decode shape."""
    from onnxruntime_amd.matmul_nbits import MatMulNBits
    M, N, K, bits, bs = 1, 2048, 1024, 4, 32
    g, _ = _mats(M, N, K, bits, bs, np.float16, True, 31)
    u, _ = _mats(M, N, K, bits, bs, np.float16, True, 32)
    op = MatMulNBitsMlp(K, N, bits, bs)
    op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), dev(u.bias))
    y = op.Compute(dev(g.A)).float()
    outs = []
    for c in (g, u):
        m = MatMulNBits(K, N, bits, bs, has_bias=True)
        m.PrePack(dev(c.B), dev(c.scales))
        outs.append(m.Compute(dev(g.A), bias=dev(c.bias)).float())
    ref = torch.nn.functional.silu(outs[0]) * outs[1]
    torch.cuda.synchronize()
    # the unfused route narrows gate and up to fp16 first: 2^-11 relative each
    assert torch.allclose(y, ref, rtol=4e-3, atol=4e-3 * float(ref.abs().max()) * 1e-2)


# ------------------------------------------------------------------------------------------------ QKV
QKV_CASES = [
    # M, Nq, Nkv, K, bits, bs
    (1, 64, 16, 128, 4, 32), (1, 4096, 1024, 4096, 4, 32), (5, 100, 24, 96, 4, 16), (16, 48, 40, 256, 8, 64),
    (33, 128, 32, 512, 4, 128), (100, 72, 8, 200, 4, 32), (300, 512, 128, 256, 4, 32), (600, 768, 256, 512, 8, 32),
    (1024, 4000, 2040, 1024, 4, 32),   # tile GEMM; outputs begin inside a wavefront's 64-column block
    (2, 6100, 2040, 512, 4, 128),      # decode with 48-column slabs: slabs straddle the borders between Q, K and V
]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("norm", [None, "simplified", "skip"])
@pytest.mark.parametrize("M,Nq,Nkv,K,bits,bs", QKV_CASES)
def test_qkv_parity(oracle, dtype, norm, M, Nq, Nkv, K, bits, bs):
    q, qm = _mats(M, Nq, K, bits, bs, dtype, True, 41)
    k, km = _mats(M, Nkv, K, bits, bs, dtype, False, 42)
    v, vm = _mats(M, Nkv, K, bits, bs, dtype, True, 43)
    op = MatMulNBitsQkv(K, Nq, Nkv, bits, bs, epsilon=1e-6, dtype=tdtype(dtype))
    assert op.PrePack(dev(q.B), dev(q.scales), dev(q.bias), dev(k.B), dev(k.scales), None, dev(v.B), dev(v.scales),
                      dev(v.bias))
    skip, gamma = _norm_inputs(M, K, dtype, M if norm == "skip" else 0, 44)
    if norm is None:
        outs = op.Compute(dev(q.A))
        act = q.A
    else:
        outs = op.Compute(dev(q.A), skip=dev(skip), norm_scale=dev(gamma), want_skip_sum=norm == "skip")
        act = simplified_layer_norm(dev(q.A), dev(gamma), 1e-6, skip=dev(skip)).cpu().numpy()
        want_act = oracle.C.simplified_layer_norm(q.A, skip, gamma, 1e-6)
        assert _ulps(act, want_act).max() <= (1 if dtype == np.float16 else 64)
        if norm == "skip":
            assert np.array_equal(outs[3].cpu().numpy(),
                                  (q.A.astype(np.float32) + skip.astype(np.float32)).astype(dtype))
    torch.cuda.synchronize()
    for got, c, n in zip(outs[:3], (q, k, v), (Nq, Nkv, Nkv)):
        got = got.cpu().numpy()
        assert got.shape == (M, n)
        y64, bound = oracle.C.matmul_f64(act, c.B, c.scales, None, c.bias, n, K, bits, bs, nthreads=8)
        err = np.abs(got.astype(np.float64) - y64)
        if dtype == np.float32:
            assert float(np.max(err / (bound + 1e-30))) <= FP32_GATE
        else:
            assert float(np.linalg.norm(err) / max(np.linalg.norm(y64), 1e-30)) <= FP16_GATE
            want = oracle.C.matmul(act, c.B, c.scales, None, c.bias, n, K, bits, bs, nthreads=8)
            assert float(np.linalg.norm(got.astype(np.float64) - want.astype(np.float64)) /
                         max(np.linalg.norm(want.astype(np.float64)), 1e-30)) <= 1e-3


@pytest.mark.parametrize("M,N,K,bits,bs", [(64, 14336, 1024, 4, 128), (20, 10500, 1024, 8, 64)])
def test_mlp_on_the_shared_activations_variant(oracle, M, N, K, bits, bs):
    """Gate and up packed as one matrix of 2 N columns wide enough for the streaming kernel's variant that shares the
    activations through LDS: the operator's output against the oracle, and against the two separate products."""
    lib = _lib.load()
    if lib.MnbGemmKernelName(M, 2 * ((N + 15) // 16 * 16), K, bits, bs, _lib.DTYPE_FLOAT16) != b"mnb_mid_shared_kernel":
        pytest.skip("this device's compute-unit count does not select the shared-activations variant here")
    g, _ = _mats(M, N, K, bits, bs, np.float16, True, 71)
    u, _ = _mats(M, N, K, bits, bs, np.float16, True, 72)
    op = MatMulNBitsMlp(K, N, bits, bs)
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), dev(u.bias))
    y = op.Compute(dev(g.A))
    torch.cuda.synchronize()
    _check_mlp(oracle, y.cpu().numpy(), g.A, g, u, N, K, bits, bs, np.float16)


def test_tile_gemm_shape_with_unaligned_output_takes_the_streaming_kernel(oracle):
    """Where the shape selects the tile GEMM but Y does not allow 16-byte stores, the streaming kernel (whose scratch
    the workspace contract reserves) writes the outputs: same result, up to the narrowing of gate / up."""
    import ctypes
    lib = _lib.load()
    M, N, K, bits, bs = 2048, 2048, 1024, 4, 32
    g, _ = _mats(M, N, K, bits, bs, np.float16, True, 51)
    u, _ = _mats(M, N, K, bits, bs, np.float16, False, 52)
    op = MatMulNBitsMlp(K, N, bits, bs)
    op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), None)
    a = dev(g.A)
    y_ref = op.Compute(a)
    wsz = lib.MnbMlpWorkspaceSize(M, N, K, bits, bs, _lib.DTYPE_FLOAT16, 0)
    assert wsz > 0
    ws = torch.empty(wsz, dtype=torch.uint8, device="cuda")
    raw = torch.zeros(M * N + 4, dtype=torch.float16, device="cuda")
    y = raw[4:].view(M, N)   # 8 bytes off a 16-byte boundary
    _lib.check(lib.MnbMlpGemm(M, N, K, bits, bs, _lib.DTYPE_FLOAT16, a.data_ptr(), K, None, op.packed.data_ptr(), 0,
                              y.data_ptr(), N, ws.data_ptr(), wsz, None))
    torch.cuda.synchronize()
    assert not raw[:4].any()
    d = (y.float() - y_ref.float()).abs()
    assert float(d.max()) <= 4e-3 * float(y_ref.float().abs().max())
    _check_mlp(oracle, y.cpu().numpy(), g.A, g, u, N, K, bits, bs, np.float16)


# ------------------------------------------------------------------------------------------------ contract
def test_fused_argument_errors():
    lib = _lib.load()
    op = MatMulNBitsMlp(256, 64, 4, 32)
    with pytest.raises(_lib.MnbError, match="activation 'gelu' is not supported"):
        MatMulNBitsMlp(256, 64, 4, 32, activation="gelu")
    g, _ = _mats(1, 64, 256, 4, 32, np.float16, False, 1)
    op.PrePack(dev(g.B), dev(g.scales), None, dev(g.B), dev(g.scales), None)
    with pytest.raises(_lib.MnbError, match="norm_scale input must be present when skip input is provided"):
        op.Compute(dev(g.A), skip=dev(g.A))
    with pytest.raises(_lib.MnbError, match="skip input must be present when input_skip_bias_sum output is requested"):
        op.Compute(dev(g.A), norm_scale=dev(np.ones(256, np.float16)), want_skip_sum=True)
    with pytest.raises(_lib.MnbError, match="norm_scale shape must be"):
        op.Compute(dev(g.A), norm_scale=dev(np.ones(255, np.float16)))
    # too small a workspace is an error, not a fault
    n = _lib.MnbNormPrologue()
    gamma = dev(np.ones(256, np.float16))
    n.norm_scale_dev, n.epsilon = gamma.data_ptr(), 1e-5
    y = torch.empty(1, 64, dtype=torch.float16, device="cuda")
    import ctypes
    rc = lib.MnbMlpGemm(1, 64, 256, 4, 32, _lib.DTYPE_FLOAT16, dev(g.A).data_ptr(), 256, ctypes.byref(n),
                        op.packed.data_ptr(), 0, y.data_ptr(), 64, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "workspace of" in _lib.last_error()
    rc = lib.MnbMlpGemm(1, 64, 256, 4, 32, _lib.DTYPE_FLOAT16, dev(g.A).data_ptr(), 256, None, op.packed.data_ptr(), 7,
                        y.data_ptr(), 64, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "activation 7 is not supported" in _lib.last_error()
    assert lib.MnbMlpPackSize(64, 256, 3, 32, _lib.DTYPE_FLOAT16) == 0  # 3-bit: no such format
    # empty batch
    assert tuple(op.Compute(torch.empty(0, 256, dtype=torch.float16, device="cuda")).shape) == (0, 64)


def test_split_shape_with_misaligned_pointers_takes_the_streaming_kernel(oracle):
    """A shape whose tile-GEMM plan cuts tiles along K (its own workspace is then non-zero): with an A or a Y that
    does not allow 16-byte accesses the streaming kernel takes over, inside the workspace the contract reserves.
    Checked against the aligned call (tile GEMM) and, on sampled rows, against the oracle."""
    import ctypes
    lib = _lib.load()
    M, N, K, bits, bs = 2048, 512, 14336, 4, 128
    r, c, p = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.MnbGemmTilePlan(M, 2 * N, K, bits, bs, 0, _lib.DTYPE_FLOAT16, ctypes.byref(r), ctypes.byref(c), ctypes.byref(p))
    assert p.value > 1, "the case is meant to be a split shape"
    g, _ = _mats(M, N, K, bits, bs, np.float16, True, 61)
    u, _ = _mats(M, N, K, bits, bs, np.float16, False, 62)
    op = MatMulNBitsMlp(K, N, bits, bs)
    op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), None)
    a = dev(g.A)
    y_ref = op.Compute(a)
    wsz = lib.MnbMlpWorkspaceSize(M, N, K, bits, bs, _lib.DTYPE_FLOAT16, 0)
    ws = torch.empty(wsz, dtype=torch.uint8, device="cuda")
    a_raw = torch.zeros(M * K + 4, dtype=torch.float16, device="cuda")
    a_off = a_raw[4:].view(M, K)
    a_off.copy_(a)
    y_raw = torch.zeros(M * N + 4, dtype=torch.float16, device="cuda")
    y_off = y_raw[4:].view(M, N)
    y_al = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    rows = np.array([0, 1, 255, 256, 1000, 2047])
    for a_t, y_t in ((a_off, y_al), (a, y_off), (a_off, y_off)):
        y_t.zero_()
        _lib.check(lib.MnbMlpGemm(M, N, K, bits, bs, _lib.DTYPE_FLOAT16, a_t.data_ptr(), K, None,
                                  op.packed.data_ptr(), 0, y_t.data_ptr(), N, ws.data_ptr(), wsz, None))
        torch.cuda.synchronize()
        assert not y_raw[:4].any()
        d = (y_t.float() - y_ref.float()).abs()
        assert float(d.max()) <= 4e-3 * float(y_ref.float().abs().max())
        _check_mlp(oracle, y_t.cpu().numpy()[rows], g.A[rows], g, u, N, K, bits, bs, np.float16)
