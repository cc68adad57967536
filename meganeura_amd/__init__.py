"""MI355X-native quantized (Q4/Q8) matmul path behind meganeura's operator surface."""
