"""Single-GPU MoE layer and its kernels behind picotron's expert_parallel module names."""
