"""MI355X-native quantized Mixture-of-Experts expert path: routing, permutation by expert, block-scaled
grouped GEMMs with a fused SwiGLU epilogue, and the weighted combine, as hand-written HIP kernels for
gfx950 behind a C-ABI library, under the reference's MoE layer and quantized-weight API."""
