"""Context-parallel ring attention (GQA/MHA and MLA variants) on HIP kernels."""
