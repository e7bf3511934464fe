"""oxidize_amd — MI355X-native quantized matvec/matmul behind oxidize-c's matvec API."""
