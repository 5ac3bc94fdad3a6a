"""MI355X-native quantized matmul for cogni-ml's GGUF path (Python-side binding of the C ABI)."""
