"""candle_amd: MI355X-native quantized matmul for candle's QMatMul path.

`candle_amd.qhip` binds the C ABI of libcandle_qhip.so (include/candle_qhip.h);
`candle_amd.quantized` mirrors candle_core::quantized's QTensor / QMatMul surface on top of it.
"""
__all__ = ["qhip", "quantized", "build"]
