from .Arch import Arch


class MI355X(Arch):
    """AMD Instinct MI355X (CDNA4, gfx950).

    The attribute names the solver and the cost model read are the reference's
    (arch/H20.py:14-60, arch/H100.py:96-119) so that the ranking code keeps its
    shape; their values are CDNA4's.  "sm" means compute unit, "warp" means a
    64-lane wavefront, "smem" means LDS.  `configure_device` overwrites the
    counts that the runtime reports (reference: arch/H20.py:69-82).
    """

    def __init__(self, para_opt=True):
        self.name = "AMD Instinct MI355X"
        self.gcn_arch = "gfx950"
        self.global_mem_capacity = "288GB"
        self.para_opt = para_opt

        # ---- execution resources -------------------------------------------------
        self.warp_size = 64
        self.num_xcd = 8  # accelerator complex dies, each with a private L2
        self.simds_per_cu = 4
        self._set_cu_count(256)
        self.max_waves_per_simd = 8
        self.max_resident_warps_per_sm = self.max_waves_per_simd * self.simds_per_cu
        self.max_resident_blocks_per_sm = 32
        self.max_threads_per_block = 1024
        # Unified register file: 512 32-bit registers per lane and SIMD, split
        # between architectural VGPRs and accumulation VGPRs (each at most 256),
        # allocated in blocks of 8.
        self.vgprs_per_simd = 512
        self.max_arch_vgprs = 256
        self.max_acc_vgprs = 256
        self.vgpr_granule = 8
        # 32-bit registers per CU (4 SIMDs x 512 x 64 lanes); the reference's
        # name for the register-file capacity.
        self.max_registers_per_sm = self.simds_per_cu * self.vgprs_per_simd * self.warp_size
        self.reg_cap = [self.max_registers_per_sm, 512]

        # ---- LDS -----------------------------------------------------------------
        self.lds_per_cu = 160 * 1024
        # One workgroup may use the whole LDS; there is no L1 carve-out.
        self.max_dyn_smem_per_block = 160 * 1024
        self.shared_mem_config_options = [160]
        self.smem_cap = [self.max_dyn_smem_per_block]
        self.smem_bank_size = 4
        self.bank_number = 64
        self.sm_clock_hz = 2.4e9
        # 128 B/clk/CU for 32/64-bit accesses; ds_read_b128 reaches 256 B/clk.
        self.lds_bytes_per_clk = 128
        self.lds_b128_bytes_per_clk = 256
        self.smem_bw_per_sm = self.lds_b128_bytes_per_clk * self.sm_clock_hz

        # ---- memory system -------------------------------------------------------
        self.dram_bw = 8000  # GB/s, HBM3E
        self.l2_bytes = 8 * 4 * 1024 * 1024  # 4 MiB per XCD
        self.l2_bytes_per_xcd = 4 * 1024 * 1024
        self.mall_bytes = 256 * 1024 * 1024  # Infinity Cache in front of HBM
        self.l2_bw = 16000  # GB/s aggregate over the 8 L2s (approximate)
        self.mall_bw = 14000  # GB/s (approximate)
        # Latency under load for Little's law in the row-wise cost model.
        self.dram_latency_s = 2.0e-6
        self.transaction_size = [64]

        # ---- compute peaks (GFLOPS) ------------------------------------------------
        # Vector fp32 (packed): 256 CU x 256 FLOP/clk x 2.4 GHz.
        self.peak_flops = 157286
        # Dense MFMA fp16/bf16 with fp32 accumulation: 256 CU x 4096 FLOP/clk x 2.4 GHz.
        self.mfma_flops_per_clk_cu = 4096
        self.peak_tc_flops = 2516582
        self.peak_tc_flops_fp32acc = self.peak_tc_flops
        # The reference's name for "the matrix-unit peak the GEMM and attention
        # kernels are judged against" (arch/H20.py:39).
        self.peak_mma_sync_flops = self.peak_tc_flops
        self.peak_mma_sync_f16acc_flops = self.peak_tc_flops

        # ---- fitted penalties read via getattr by the cost model ---------------------
        self.gemm_excess_stage_penalty = 0.02
        self.gemm_fill_latency_s = 0.75e-6
        self.fa_cta_sync_penalty = 0.05

        self.bandwidth = [self.dram_bw, self.smem_bw_per_sm * self.sm_nums / 1e9]
        self.compute_capability = "gfx950"

    def _set_cu_count(self, n: int):
        self.sm_nums = n
        self.compute_max_core = [n]
        self.mem_max_core = [n]
        self.compute_sm_partition = [n, self.simds_per_cu]
        self.smem_sm_partition = [n, self.simds_per_cu]
        self.cus_per_xcd = max(1, n // self.num_xcd)

    def configure_device(self, info):
        """Specialises the model with a `DeviceInfo` read through the HIP driver."""
        self.name = info.name or self.name
        self.gcn_arch = info.gcn_arch.split(":")[0] or self.gcn_arch
        if info.cu_count > 0:
            self._set_cu_count(info.cu_count)
        if info.clock_khz > 0:
            self.sm_clock_hz = info.clock_khz * 1e3
        if info.lds_per_block > 0:
            self.max_dyn_smem_per_block = int(info.lds_per_block)
            self.smem_cap = [self.max_dyn_smem_per_block]
        if info.total_mem > 0:
            self.global_mem_capacity = f"{info.total_mem / 2**30:.0f}GiB"
        self.smem_bw_per_sm = self.lds_b128_bytes_per_clk * self.sm_clock_hz
        self.peak_flops = self.sm_nums * 256 * self.sm_clock_hz / 1e9
        self.peak_tc_flops = self.sm_nums * self.mfma_flops_per_clk_cu * self.sm_clock_hz / 1e9
        self.peak_tc_flops_fp32acc = self.peak_tc_flops
        self.peak_mma_sync_flops = self.peak_tc_flops
        self.peak_mma_sync_f16acc_flops = self.peak_tc_flops
        self.bandwidth = [self.dram_bw, self.smem_bw_per_sm * self.sm_nums / 1e9]
        return self
