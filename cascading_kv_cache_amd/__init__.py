"""MI355X-native Cascading KV Cache attention hot path (HIP kernels behind a C ABI)."""
