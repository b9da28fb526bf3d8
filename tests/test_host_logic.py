"""CPU-side tests: the C ABI library loads and exports every declared symbol; shape validation and error text."""
import re
from pathlib import Path

import pytest

from onnxruntime_amd import _lib
from onnxruntime_amd._lib import MnbError
from onnxruntime_amd.matmul_nbits import MatMulNBits, check_inputs

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "mnb_mi355x.h").read_text()
    declared = set(re.findall(r"MNB_API\s+[\w\s\*]+?\b(Mnb\w+)\s*\(", header))
    assert len(declared) >= 14
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.MnbGetVersion() >= 1


def test_availability_and_sizes():
    lib = _lib.load()
    for bits in (2, 4, 8):
        for bs in (16, 32, 64, 128, 256):
            for dt in (_lib.DTYPE_FLOAT, _lib.DTYPE_FLOAT16):
                assert lib.MnbIsAvailable(bits, bs, dt) == 1
    assert lib.MnbIsAvailable(3, 32, _lib.DTYPE_FLOAT16) == 0
    assert lib.MnbIsAvailable(4, 512, _lib.DTYPE_FLOAT16) == 0
    assert lib.MnbIsAvailable(4, 32, 16) == 0  # bf16
    # packed size: weights (N*K/2) + fp16 scales for the headline decode shape, no padding needed
    assert lib.MnbPackQuantBDataSize(14336, 4096, 4, 128, 0, _lib.DTYPE_FLOAT16) == 14336 * 2048 + 14336 * 32 * 2
    # 2-bit weights are stored as nibbles with explicit zero points: the 4-bit size with 4-byte meta entries ...
    four = lib.MnbPackQuantBDataSize(14336, 4096, 4, 128, 1, _lib.DTYPE_FLOAT16)
    # ... plus, for fp16 models with blocks of 32 and more, a copy in their own width for the decode kernel (N*K/4)
    assert lib.MnbPackQuantBDataSize(14336, 4096, 2, 128, 0, _lib.DTYPE_FLOAT16) == four + 14336 * 4096 // 4
    assert lib.MnbPackQuantBDataSize(14336, 4096, 2, 16, 0, _lib.DTYPE_FLOAT16) == \
        lib.MnbPackQuantBDataSize(14336, 4096, 4, 16, 1, _lib.DTYPE_FLOAT16)
    assert lib.MnbPackQuantBDataSize(14336, 4096, 2, 128, 0, _lib.DTYPE_FLOAT) == \
        lib.MnbPackQuantBDataSize(14336, 4096, 4, 128, 1, _lib.DTYPE_FLOAT)
    assert lib.MnbPackQuantBDataSize(14336, 4096, 4, 32, 1, _lib.DTYPE_FLOAT16) == 14336 * 2048 + 14336 * 128 * 4
    assert lib.MnbPackQuantBDataSize(0, 4096, 4, 32, 1, _lib.DTYPE_FLOAT16) == 0


def _fails(substr, *args, **kw):
    with pytest.raises(MnbError) as e:
        check_inputs(*args, **kw)
    assert substr in str(e.value), str(e.value)
    assert e.value.code == _lib.INVALID_ARGUMENT


def test_check_inputs_messages():
    # N=8, K=32, bs=16, bits=4: B [8,2,8], scales [8,2] or [16], zp [8,1] or [8]
    check_inputs((8, 2, 8), (8, 2), (8, 1), None, (8,), 8, 32, 16, 4)
    check_inputs((8, 2, 8), (16,), (8,), None, None, 8, 32, 16, 4)          # legacy 1-D shapes
    check_inputs(None, (8, 2), None, (32,), None, 8, 32, 16, 4)            # B already packed, g_idx [K]
    _fails("bits should be 2, 4 or 8, got 3", (8, 2, 6), (8, 2), None, None, None, 8, 32, 16, 3)
    _fails("block_size must be a power of 2, and >= 16. Got 8", (8, 4, 4), (8, 4), None, None, None, 8, 32, 8, 4)
    _fails("block_size must be a power of 2, and >= 16. Got 48", (8, 1, 24), (8, 1), None, None, None, 8, 32, 48, 4)
    _fails("Input 'quantized_weight' is expected to have shape {8,2,8}, got {8,2,16}", (8, 2, 16), (8, 2), None,
           None, None, 8, 32, 16, 4)
    _fails("Input 'scales' is expected to have shape {16} or {8,2}, got {8,3}", (8, 2, 8), (8, 3), None, None, None,
           8, 32, 16, 4)
    _fails("Input 'zero_points' is expected to have shape {8} or {8,1}, got {8,2}", (8, 2, 8), (8, 2), (8, 2), None,
           None, 8, 32, 16, 4)
    _fails("Input 'bias' is expected to have shape {8}, got {9}", (8, 2, 8), (8, 2), None, None, (9,), 8, 32, 16, 4)
    _fails("Input 'group_index' is expected to have shape {30} or {32}, got {31}", (8, 2, 8), (8, 2), None, (31,),
           None, 8, 30, 16, 4)
    # typed (non-uint8) zero points: same dtype as scales, shape [N, k_blocks]
    import torch
    check_inputs((8, 2, 8), (8, 2), (8, 2), None, None, 8, 32, 16, 4, scales_dtype=torch.float16,
                 zp_dtype=torch.float16)
    _fails("should have the same data type when zero_points is not uint8", (8, 2, 8), (8, 2), (8, 2), None, None, 8,
           32, 16, 4, scales_dtype=torch.float16, zp_dtype=torch.float32)


def test_constructor_and_prepack_guards():
    import torch
    with pytest.raises(MnbError, match="Only 2b, 4b and 8b quantization is supported"):
        MatMulNBits(32, 8, bits=3)
    with pytest.raises(MnbError, match="Only block sizes 16, 32, 64, 128, and 256 are supported for MatMulNBits op, "
                                       "got: 512"):
        MatMulNBits(1024, 8, block_size=512)
    op = MatMulNBits(32, 8, bits=4, block_size=16, has_zero_points=True)
    b = torch.zeros(8, 2, 8, dtype=torch.uint8)
    s = torch.zeros(8, 2, dtype=torch.float16)
    z = torch.zeros(8, 1, dtype=torch.uint8)
    with pytest.raises(MnbError, match=r"MatMulNBits PrePack: B initializer shape \{8,2,16\} does not match "
                                       r"attribute-derived shape \[8,2,8\]"):
        op.PrePack(torch.zeros(8, 2, 16, dtype=torch.uint8), s, z)
    with pytest.raises(MnbError, match=r"MatMulNBits PrePack: scales initializer shape \{8,3\}"):
        op.PrePack(b, torch.zeros(8, 3, dtype=torch.float16), z)
    with pytest.raises(MnbError, match=r"MatMulNBits PrePack: zero_points initializer shape \{8,2\}"):
        op.PrePack(b, s, torch.zeros(8, 2, dtype=torch.uint8))
    # configurations the device path declines (they stay on the CPU provider)
    assert MatMulNBits(32, 8, bits=2, block_size=16).supported
    # the reference's "very rare" inputs run through the variant entry points, within the reference's own limits
    assert MatMulNBits(32, 8, has_g_idx=True).supported and MatMulNBits(32, 8, has_g_idx=True).variant
    assert MatMulNBits(32, 8, has_zero_points=True, zero_points_dtype=torch.float16).supported
    assert MatMulNBits(32, 8, dtype=torch.bfloat16).supported
    assert not MatMulNBits(32, 8, bits=8, has_g_idx=True).supported
    assert not MatMulNBits(32, 8, bits=8, has_zero_points=True, zero_points_dtype=torch.float16).supported
    assert not MatMulNBits(32, 8, has_zero_points=True, zero_points_dtype=torch.float32).supported  # T3 must be T1


def test_variant_plans_without_a_gpu():
    """Planning is host work: block size 16 in group order, padding, trivial group indices, the reference's limits."""
    import ctypes
    import numpy as np
    lib = _lib.load()

    def plan(N, K, bits, bs, dtype, zp_kind, g=None):
        p = _lib.MnbVariantPlan()
        gp, gl = (None, 0) if g is None else (np.ascontiguousarray(g, np.int32), len(g))
        rc = lib.MnbVariantMakePlan(N, K, bits, bs, dtype, zp_kind,
                                    None if gp is None else gp.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), gl,
                                    ctypes.byref(p))
        return rc, p

    K, bs = 200, 32
    kb = (K + bs - 1) // bs
    rc, p = plan(8, K, 4, bs, _lib.DTYPE_FLOAT16, _lib.ZP_NONE, np.arange(K) // bs)
    assert rc == 0 and not p.has_g_idx and p.packed_k == K and p.packed_block_size == bs   # trivial: dropped
    assert p.compute_dtype == _lib.DTYPE_FLOAT16
    g = np.arange(K) % kb                                                                  # groups interleaved
    rc, p = plan(8, K, 4, bs, _lib.DTYPE_FLOAT16, _lib.ZP_UINT8, g)
    counts = np.bincount(g, minlength=kb)
    assert rc == 0 and p.has_g_idx and p.packed_block_size == 16
    assert p.packed_k == int(((counts + 15) // 16 * 16).sum())
    assert p.gather_offset < p.packed_bytes
    rc, p = plan(8, K, 4, bs, _lib.DTYPE_FLOAT16, _lib.ZP_TYPED)
    assert rc == 0 and p.compute_dtype == _lib.DTYPE_FLOAT and not p.has_g_idx
    rc, p = plan(8, K, 4, bs, _lib.DTYPE_BFLOAT16, _lib.ZP_NONE)
    assert rc == 0 and p.compute_dtype == _lib.DTYPE_FLOAT
    rc, _ = plan(8, K, 4, bs, _lib.DTYPE_FLOAT, _lib.ZP_NONE, np.full(K, kb))              # group out of range
    assert rc == _lib.INVALID_ARGUMENT and "which is out of valid range [0, 7)" in _lib.last_error()
    # the padded form [k_blocks * block_size] is checked to its end, as the reference does (matmul_nbits_helper.h:92-103)
    padded = np.concatenate([np.arange(K) // bs, np.full(kb * bs - K, kb - 1)])
    rc, p = plan(8, K, 4, bs, _lib.DTYPE_FLOAT, _lib.ZP_NONE, padded)
    assert rc == 0 and not p.has_g_idx
    padded[K + 3] = -1
    rc, _ = plan(8, K, 4, bs, _lib.DTYPE_FLOAT, _lib.ZP_NONE, padded)
    assert rc == _lib.INVALID_ARGUMENT
    assert f"group_index value at index {K + 3} is -1, which is out of valid range [0, 7)" in _lib.last_error()
    rc, _ = plan(8, K, 4, bs, _lib.DTYPE_FLOAT, _lib.ZP_NONE, np.zeros(K + 1))             # wrong length
    assert rc == _lib.INVALID_ARGUMENT and "group_index" in _lib.last_error()
    rc, _ = plan(8, K, 8, bs, _lib.DTYPE_FLOAT, _lib.ZP_TYPED)
    assert rc == _lib.NOT_IMPLEMENTED and "Only 2b and 4b quantization is supported for unpacked compute" in _lib.last_error()
    rc, _ = plan(8, K, 8, bs, _lib.DTYPE_FLOAT, _lib.ZP_NONE, g)
    assert rc == _lib.NOT_IMPLEMENTED


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    lib = _lib.load()
    rc = lib.MnbGemm(1, 8, 32, 3, 16, 0, _lib.DTYPE_FLOAT16, None, 32, None, None, None, 8, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "Only 2b, 4b and 8b" in _lib.last_error()
    rc = lib.MnbGemm(1, 8, 32, 4, 48, 0, _lib.DTYPE_FLOAT16, None, 32, None, None, None, 8, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "got: 48" in _lib.last_error()
    rc = lib.MnbGemm(1, 8, 32, 4, 16, 0, 16, None, 32, None, None, None, 8, None, 0, None)   # bf16 activations
    assert rc == _lib.NOT_IMPLEMENTED
    rc = lib.MnbGemm(1, 8, 32, 4, 16, 0, _lib.DTYPE_FLOAT16, None, 32, None, None, None, 8, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "must not be NULL" in _lib.last_error()
    assert lib.MnbGemm(0, 8, 32, 4, 16, 0, _lib.DTYPE_FLOAT16, None, 32, None, None, None, 8, None, 0, None) == 0
    rc = lib.MnbPackQuantBData(8, 32, 4, 16, _lib.DTYPE_FLOAT16, None, None, None, None, None)
    assert rc == _lib.INVALID_ARGUMENT


def test_tile_gemm_offsets_stay_below_four_gib():
    """The tile GEMM adds a 32-bit per-lane byte offset to a base that holds the tile's first row and the k-step: the
    largest offset is that of row 255 of the tile, k chunk 7, last byte = (255 * lda + 63) * 2 + 1, whatever M is.
    Rows beyond 4 GiB from the start of A (M * lda * 2 >= 2^32) therefore stay reachable; a pitch that alone
    overflows 32 bits must select another kernel."""
    lib = _lib.load()
    N, K, bits, bs = 14336, 14336, 4, 32
    name = lambda M, lda: lib.MnbGemmKernelNameStrided(M, N, K, bits, bs, _lib.DTYPE_FLOAT16, lda).decode()
    largest = lambda lda: (255 * lda + 7 * 8 + 7) * 2 + 1          # exact integer arithmetic
    # M beyond the old limit (M * lda * 2 >= 2^32 at M >= 149797 for lda = 14336): offsets do not depend on M
    for M in (2048, 149796, 149797, 262144, 1 << 21):
        assert M * K * 2 < (1 << 32) or M >= 149797
        assert name(M, K) == "mnb_gemm256_kernel" and largest(K) < (1 << 32)
    # pitches around the limit: 255 * lda * 2 crosses 2^32 between lda = 8421496 and 8421504 (multiples of 8)
    limit = max(l for l in range(8421000, 8422000, 8) if largest(l) < (1 << 32))
    assert largest(limit) < (1 << 32) <= largest(limit + 8)
    assert name(2048, limit) == "mnb_gemm256_kernel"
    for lda in (limit + 8, limit + 4096, 1 << 24, 1 << 30):
        assert largest(lda) >= (1 << 32)
        assert name(2048, lda) != "mnb_gemm256_kernel"


def test_dispatch_on_the_benchmark_layer_shapes():
    """The kernel choice and the use of a split (workspace) for one Llama-3-8B layer: a guard for the calibrated plan.
    The plan's inputs are the problem and the device's CU count and clock; without a device it assumes 256 CUs at
    2.4 GHz, which is what it was calibrated on."""
    lib = _lib.load()
    if lib.MnbGetDeviceCount() > 0:
        import pytest
        pytest.skip("device properties replace the defaults the expectations below were written for")
    from onnxruntime_amd.synthetic import C5_SHAPES
    want = {  # M -> kernel, whether the tile GEMM splits tiles along K
        # (qkv at M = 256: 48 slabs x 4 row blocks = 192 workgroups, one round: activations shared through LDS)
        "qkv": {1: ("skinny", 0), 64: ("mid", 1), 256: ("mid_shared", 1), 1024: ("gemm256", 0), 4096: ("gemm256", 0)},
        # (o at M = 1024: 128 x 128 tiles, one per compute unit, instead of a cut along K)
        "o": {1: ("skinny", 0), 64: ("mid", 1), 256: ("mid", 1), 1024: ("gemm256", 0), 4096: ("gemm256", 0)},
        # (gate+up at M = 64: 224 slabs of 128 columns, one round of workgroups: activations shared through LDS)
        "gate_up": {1: ("skinny", 0), 64: ("mid_shared", 1), 256: ("gemm256", 0), 1024: ("gemm256", 0), 4096: ("gemm256", 0)},
        "down": {1: ("skinny", 0), 64: ("mid", 1), 256: ("mid", 1), 1024: ("gemm256", 1), 4096: ("gemm256", 0)},
    }
    for bits, bs in ((4, 128), (8, 64)):
        for name, (K, N) in C5_SHAPES.items():
            for M, (kernel, ws) in want[name].items():
                got = lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16).decode()
                assert got == f"mnb_{kernel}_kernel", (bits, name, M, got)
                need = lib.MnbGemmWorkspaceSize(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16)
                assert (need > 0) == bool(ws), (bits, name, M, need)
    import ctypes
    r, c, p = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    plan = lambda M, N, K: (lib.MnbGemmTilePlan(M, N, K, 4, 128, 1, _lib.DTYPE_FLOAT16, ctypes.byref(r), ctypes.byref(c),
                                                ctypes.byref(p)), r.value, c.value, p.value)[1:]
    assert plan(1024, 4096, 4096) == (128, 128, 1)      # o
    assert plan(1024, 4096, 14336) == (128, 256, 2)     # down
    assert plan(4096, 28672, 4096) == (256, 256, 1)     # gate_up
    assert plan(64, 4096, 4096) == (0, 0, 0)            # another kernel


def test_fused_workspace_covers_the_streaming_kernel_on_split_shapes():
    """Where the tile GEMM's plan cuts tiles along K its own workspace is non-zero; the fused operators' workspace
    must still hold the streaming kernel's copy of A, which takes over when pointers turn out to be misaligned."""
    import ctypes
    lib = _lib.load()
    # the streaming kernel's copy of A (4-bit weights): chunks of 128 k, 16-row tiles in blocks of four, 4 KiB each
    mid_bytes = lambda M, K: -(-K // 128) * 4 * (-(-M // 64) * 4) * 64 * 16  # noqa: E731
    assert lib.MnbGemmKernelName(64, 256, 4096, 4, 128, _lib.DTYPE_FLOAT16) == b"mnb_mid_kernel"
    assert lib.MnbGemmWorkspaceSize(64, 256, 4096, 4, 128, 0, _lib.DTYPE_FLOAT16) == mid_bytes(64, 4096)
    r, c, p = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    seen = 0
    for M in (512, 1024, 2048, 4096):
        for N in (256, 512, 1024, 2048):
            for K in (8192, 14336):
                Np = 2 * N
                lib.MnbGemmTilePlan(M, Np, K, 4, 128, 0, _lib.DTYPE_FLOAT16, ctypes.byref(r), ctypes.byref(c),
                                    ctypes.byref(p))
                if p.value <= 1:
                    continue
                seen += 1
                split = lib.MnbGemmWorkspaceSize(M, Np, K, 4, 128, 0, _lib.DTYPE_FLOAT16)
                mid = mid_bytes(M, K)
                need = lib.MnbMlpWorkspaceSize(M, N, K, 4, 128, _lib.DTYPE_FLOAT16, 0)
                assert split > 0 and need >= max(split, mid), (M, N, K, split, mid, need)
    assert seen >= 8


def test_int8_route_sizes_agree_with_what_the_kernel_accepts():
    """MnbGemmInt8WorkspaceSize is 0 exactly where MnbGemmInt8 declines, so callers that ask first fall back to the
    full-accuracy route instead of running into an error: blocks of 32, and activations whose scales and sums lie
    beyond the kernel's 32-bit offsets (2 * ceil(K / bs) * roundup(M, 128) * 4 bytes must stay below 4 GiB)."""
    lib = _lib.load()
    f16 = _lib.DTYPE_FLOAT16
    assert lib.MnbGemmInt8WorkspaceSize(64, 256, 512, 4, 64, 0, f16) > 0
    assert lib.MnbGemmInt8WorkspaceSize(64, 256, 512, 4, 32, 0, f16) == 0
    K, bs = 1 << 20, 64                      # 16384 blocks per row
    m_ok, m_big = 32640, 32768               # 2 * 16384 * M * 4 < 2^32  <=>  M < 32768
    assert lib.MnbGemmInt8WorkspaceSize(m_ok, 256, K, 4, bs, 0, f16) > 0
    assert lib.MnbGemmInt8WorkspaceSize(m_big, 256, K, 4, bs, 0, f16) == 0
    assert lib.MnbGemmInt8(m_big, 256, K, 4, bs, 0, f16, 256, K, 256, None, 256, 256, 256, 1 << 40, None) == _lib.NOT_IMPLEMENTED
    assert "M * K / block_size below 2^29" in _lib.last_error()
