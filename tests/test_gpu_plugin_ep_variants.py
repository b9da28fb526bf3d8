"""A group index, zero points in the activation type and bfloat16 activations through the plugin EP: GetCapability
claims such nodes when everything the packed buffer depends on is a constant initializer, PrePack plans and packs the
transformed problem (g_idx arrives in host memory: the kernel definition asks for that input on the CPU), Compute runs
the library's variant GEMM.  Expected values: float64 product over the oracle's restatement of the reference's
dequantiser for these inputs (matmul_nbits_impl.cc:19-75)."""
import numpy as np
import pytest

from ep_host import host
from oracle import oracle
from test_gpu_variants import make, check as check_tensor

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not host.available(), reason="plugin EP or host shim not built")]

C = oracle.C


def _as_tensor(y):
    """numpy result (bfloat16 as uint16 bit patterns) -> the torch tensor the checker of test_gpu_variants takes."""
    import torch
    return torch.from_numpy(y.view(np.int16)).view(torch.bfloat16) if y.dtype == np.uint16 else torch.from_numpy(y)


def _run(c, N, K, bits, bs, **kw):
    return host.run_matmul_nbits(N, K, bits, bs, c["A"], c["B"], c["scales"], c["zp"], c["g"], c["bias"],
                                 constant=kw.pop("constant", ("B", "scales", "zero_points", "g_idx", "bias")), **kw)


@pytest.mark.parametrize("kind,zp_kind,g_kind", [("f32", "typed", "none"), ("f16", "typed", "none"),
                                                 ("f16", "u8", "act_order"), ("f32", "none", "ragged"),
                                                 ("f16", "typed", "ragged"), ("bf16", "none", "none"),
                                                 ("bf16", "typed", "act_order"), ("f16", "none", "trivial")])
@pytest.mark.parametrize("M", [1, 48])
def test_variants_through_plugin(kind, zp_kind, g_kind, M):
    N, K, bs = 136, 288, 32
    c = make(kind, N, K, 4, bs, zp_kind, g_kind, M, seed=M + len(g_kind), bias=True)
    y, trace = _run(c, N, K, 4, bs, repeat=2)
    assert "claimed=1" in trace
    want = "prepacked=1,2," + ("3," if c["zp"] is not None else "") + ("4," if c["g"] is not None else "")
    assert want in trace, trace
    check_tensor(kind, c, _as_tensor(y), N, K, 4, bs)


def test_two_bit_typed_zero_points_through_plugin():
    N, K, bs = 40, 128, 16
    c = make("f16", N, K, 2, bs, "typed", "none", 3, seed=3)
    y, _ = _run(c, N, K, 2, bs)
    check_tensor("f16", c, _as_tensor(y), N, K, 2, bs)


def test_errors_surface_at_prepack():
    N, K, bs = 16, 64, 32
    c = make("f32", N, K, 4, bs, "none", "ragged", 2, seed=1)
    c["g"][5] = 2
    with pytest.raises(host.EpHostError) as e:
        _run(c, N, K, 4, bs)
    assert e.value.code == 2 and "group_index value at index 5 is 2, which is out of valid range [0, 2)" in e.value.message
    c = make("f16", N, K, 4, bs, "typed", "none", 2, seed=1)
    c["zp"] = c["zp"][:, :1]
    with pytest.raises(host.EpHostError) as e:
        _run(c, N, K, 4, bs)
    assert e.value.code == 2 and "zero_points" in e.value.message
