"""MI355X-native com.microsoft::MatMulNBits: HIP kernels behind a C ABI, plus the host mirror of the operator."""
from ._lib import MnbError, LIB_PATH  # noqa: F401


def __getattr__(name):
    if name in ("MatMulNBits", "check_inputs", "dequantize_blockwise", "dequantize_blockwise_variant", "quantize_blockwise",
                "MatMulNBitsMlp",
                "MatMulNBitsQkv", "simplified_layer_norm"):
        from . import matmul_nbits
        return getattr(matmul_nbits, name)
    raise AttributeError(name)
