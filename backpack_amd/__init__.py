"""backpack_amd — MI355X-native GGUF k-quant fused dequant-matmul.

`capi` binds the C ABI (include/bpk_kquant.h); `kquant` is the host-side op
layer over torch device tensors; `synth` generates the benchmark workloads."""
