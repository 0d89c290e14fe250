"""Host side of the MI355X paged-attention path: counterparts of the reference's
``mini_sglang_mlx.attention.backend`` and ``mini_sglang_mlx.kvcache.mha_pool`` on torch-ROCm,
plus the seeded synthetic workloads and roofline arithmetic used by tests and bench."""
