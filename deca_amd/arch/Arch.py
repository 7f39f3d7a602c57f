class Arch:
    """Attribute bag describing one GPU; the solver and the cost model read
    plain attributes (reference: arch/Arch.py:1-43, whose accessors serve the
    legacy two-level tiling path only)."""

    name = "generic"
    bandwidth = [0.0, 0.0]  # GB/s: [DRAM, LDS aggregate]
    peak_flops = 0.0  # GFLOPS, vector fp32

    def memory_bw(self, mem_level: int) -> float:
        return self.bandwidth[mem_level]

    def describe(self) -> str:
        keys = (
            "name", "sm_nums", "num_xcd", "sm_clock_hz", "warp_size", "lds_per_cu",
            "max_dyn_smem_per_block", "vgprs_per_simd", "max_waves_per_simd", "dram_bw",
            "l2_bytes", "mall_bytes", "peak_mma_sync_flops", "peak_flops",
        )
        return ", ".join(f"{k}={getattr(self, k, None)}" for k in keys)
