"""Kernel specialisations the GPU tests use, listed in one place so that the
build step can compile all of them ahead of the GPU run."""

from deca_amd.kernels.flash_attn_hip import FAConfig, make_flash_attn_fwd
from deca_amd.kernels.gemm_hip import GemmConfig, make_gemm_tc
from deca_amd.kernels.rowwise_hip import RowConfig, make_rowwise

# (op, M, N, dtype, cfg)
ROWWISE_CASES = [
    # reg mode, the benchmark row lengths at a CPU-checkable row count
    ("softmax", 256, 4096, "float16", RowConfig(128, 1, 8)),
    ("softmax", 256, 4096, "float16", RowConfig(64, 1, 8)),
    ("softmax", 256, 4096, "float16", RowConfig(256, 2, 8)),
    ("softmax", 256, 4096, "float16", RowConfig(512, 2, 8, hint=True)),
    ("softmax", 256, 4096, "bfloat16", RowConfig(128, 2, 8)),
    ("softmax", 256, 4096, "float16", RowConfig(128, 4, 4)),
    ("softmax", 256, 4096, "float16", RowConfig(1024, 1, 4)),
    # rows owned by a slice of a wave
    ("softmax", 512, 256, "float16", RowConfig(16, 8, 8)),
    ("softmax", 512, 1024, "float16", RowConfig(32, 4, 8)),
    # ragged rows: the last chunk is out of the row for the upper lanes
    ("softmax", 128, 1000, "float16", RowConfig(64, 2, 8)),
    ("softmax", 128, 4104, "bfloat16", RowConfig(128, 1, 8)),
    ("softmax", 64, 32000, "float16", RowConfig(256, 1, 8, "twopass", 4)),
    ("softmax", 64, 32000, "float16", RowConfig(1024, 1, 8, "twopass", 2, True)),
    ("softmax", 64, 32000, "float16", RowConfig(1024, 1, 8, "reg")),
    ("softmax", 16, 128256, "bfloat16", RowConfig(1024, 1, 8, "twopass", 4)),
    # lean reg mode: a vocabulary-size row cached in registers (only the packed row
    # survives between the passes), and a short row over very few lanes
    ("softmax", 32, 128256, "float16", RowConfig(1024, 1, 8, "reg", 1, True)),
    ("softmax", 32, 128256, "bfloat16", RowConfig(512, 1, 8, "reg")),
    ("rmsnorm", 32, 128256, "bfloat16", RowConfig(1024, 1, 8, "reg", 1, True)),
    ("rmsnorm", 32, 128256, "float16", RowConfig(512, 1, 8, "reg")),
    ("softmax", 512, 4096, "float16", RowConfig(16, 8, 8)),
    ("softmax", 256, 4096, "float16", RowConfig(64, 4, 8, "twopass", 2)),
    ("softmax", 256, 4096, "float16", RowConfig(128, 1, 4, "twopass", 1, True)),
    # single-row and single-block extremes
    ("softmax", 4, 128, "float16", RowConfig(16, 4, 8)),
    ("rmsnorm", 256, 4096, "bfloat16", RowConfig(128, 1, 8)),
    ("rmsnorm", 256, 4096, "bfloat16", RowConfig(64, 2, 8, hint=True)),
    ("rmsnorm", 256, 4096, "float16", RowConfig(256, 1, 8)),
    ("rmsnorm", 256, 8192, "float16", RowConfig(512, 1, 8)),
    ("rmsnorm", 256, 8192, "float16", RowConfig(1024, 1, 8)),
    ("rmsnorm", 256, 8192, "float16", RowConfig(128, 2, 4)),
    ("rmsnorm", 128, 1000, "bfloat16", RowConfig(64, 2, 8)),
    ("rmsnorm", 512, 1024, "float16", RowConfig(32, 2, 8)),
    ("rmsnorm", 256, 4096, "bfloat16", RowConfig(64, 4, 8, "twopass", 2)),
    ("rmsnorm", 64, 32000, "float16", RowConfig(512, 2, 8, "twopass", 4, True)),
]

# Full-size benchmark shapes (property checks + a sampled comparison).
ROWWISE_FULL = [
    ("softmax", 16384, 4096, "float16", RowConfig(128, 1, 8)),
    ("rmsnorm", 16384, 4096, "bfloat16", RowConfig(128, 1, 8)),
    ("rmsnorm", 8192, 8192, "float16", RowConfig(256, 1, 8)),
]


def rowwise_specs(eps: float = 1e-6):
    return [make_rowwise(op, M, N, dt, cfg, eps) for op, M, N, dt, cfg in ROWWISE_CASES + ROWWISE_FULL]


# (M, N, K, cfg): sizes the CPU checker finishes in seconds
GEMM_CASES = [
    # direct-to-LDS ring: (BM, BN, BK, wm, wn, stages, raster, epi_smem, xcd, direct)
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 128, 2, 1, False, False, True)),
    (512, 512, 512, GemmConfig(256, 256, 32, 128, 128, 3, 2, True, False, True)),
    (512, 1024, 256, GemmConfig(256, 256, 32, 128, 128, 4, 2, False, True, True)),
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, False, False, True)),
    (512, 512, 512, GemmConfig(256, 256, 32, 64, 128, 4, 1, True, False, True)),
    (512, 512, 512, GemmConfig(128, 128, 64, 64, 64, 3, 4, False, True, True)),
    (512, 512, 512, GemmConfig(128, 128, 32, 64, 32, 4, 4, True, True, True)),
    (384, 640, 1088, GemmConfig(128, 128, 64, 64, 64, 2, 1, False, False, True)),
    (512, 512, 2048, GemmConfig(128, 256, 64, 64, 128, 3, 2, False, True, True)),
    (256, 256, 128, GemmConfig(64, 64, 64, 32, 32, 2, 1, False, False, True)),
    (128, 192, 64, GemmConfig(64, 64, 32, 32, 64, 2, 2, False, False, True)),
    (1024, 1024, 512, GemmConfig(256, 256, 32, 128, 128, 3, 4, False, True, True)),
    # raster 0: an 8 x 4 sub-block of tiles per XCD, 8 neighbours in flight (one round; four
    # rounds; an odd number of sub-block rows; with the tail split)
    (3072, 4096, 128, GemmConfig(128, 128, 64, 64, 64, 2, 0, False, True, True)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 0, True, True, True, True)),
    (1024, 1024, 128, GemmConfig(64, 64, 64, 32, 32, 2, 0, False, True, True)),
    (2048, 2048, 64, GemmConfig(64, 64, 32, 32, 64, 2, 0, True, True, True)),
    # tail: the 64 tiles of the partial last wave (576 = 512 + 64) as 256 quarter tiles
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 4, True, True, True, True)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 1, False, True, True, True)),
    # 16x16x32 MFMA body: ring depths 2..5, one or two k-steps per K-tile, both wave
    # orientations, the barrier before or inside the last k-step, both epilogues, the block
    # order and the tail split
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16)),
    (512, 512, 512, GemmConfig(256, 256, 64, 64, 128, 2, 2, False, False, True, mfma=16, early=2)),
    (512, 1024, 256, GemmConfig(256, 256, 32, 128, 64, 3, 2, True, True, True, mfma=16, early=4)),
    (512, 512, 512, GemmConfig(256, 256, 32, 128, 64, 4, 1, False, False, True, mfma=16)),
    (512, 512, 512, GemmConfig(256, 256, 32, 64, 128, 5, 1, True, False, True, mfma=16, early=3)),
    (512, 512, 512, GemmConfig(128, 128, 64, 64, 64, 3, 4, False, True, True, mfma=16, early=1)),
    (384, 640, 1088, GemmConfig(128, 128, 64, 64, 32, 4, 1, True, False, True, mfma=16)),
    (256, 256, 128, GemmConfig(64, 64, 64, 32, 32, 2, 1, False, False, True, mfma=16)),
    (128, 192, 64, GemmConfig(64, 64, 32, 32, 64, 2, 2, False, False, True, mfma=16)),
    (3072, 4096, 128, GemmConfig(128, 128, 64, 64, 64, 2, 0, False, True, True, mfma=16, early=2)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 0, True, True, True, True, mfma=16)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 4, True, True, True, True, mfma=16, early=2)),
    # ... with the accumulators tied to accumulation registers: the large and the small wave
    # tiles, one k-step per K-tile, deep rings, the barrier inside the last k-step, the tail
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16, agpr=True)),
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 2, False, False, True, mfma=16, early=4, agpr=True)),
    (512, 1024, 256, GemmConfig(128, 128, 32, 64, 32, 4, 2, True, True, True, mfma=16, agpr=True)),
    (384, 640, 1088, GemmConfig(128, 128, 64, 64, 32, 5, 1, True, False, True, mfma=16, early=2, agpr=True)),
    (256, 256, 128, GemmConfig(64, 64, 64, 32, 32, 2, 1, False, False, True, mfma=16, agpr=True)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 0, True, True, True, True, mfma=16, agpr=True)),
    # ... with the tile loads dealt over the MFMA groups (`spread`): windows shorter and longer
    # than the groups behind the barrier, rings of 2..5, one k-step per K-tile (two tiles per
    # loop iteration), builtin and accumulation-register MFMAs, the block order and the tail
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16, early=4, agpr=True, spread=6)),
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 2, False, False, True, mfma=16, spread=2)),
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16, early=6, spread=15)),
    (512, 1024, 256, GemmConfig(256, 256, 32, 128, 64, 3, 2, True, True, True, mfma=16, early=4, spread=6)),
    (512, 512, 512, GemmConfig(256, 256, 32, 64, 128, 5, 1, True, False, True, mfma=16, early=3, spread=3)),
    (384, 640, 1088, GemmConfig(128, 128, 64, 64, 32, 4, 1, True, False, True, mfma=16, early=2, agpr=True, spread=3)),
    (256, 256, 128, GemmConfig(64, 64, 64, 32, 32, 2, 1, False, False, True, mfma=16, spread=3)),
    (128, 192, 64, GemmConfig(64, 64, 32, 32, 64, 2, 2, False, False, True, mfma=16, spread=1)),
    (3072, 4096, 128, GemmConfig(128, 128, 64, 64, 64, 2, 0, False, True, True, mfma=16, early=2, spread=3)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 0, True, True, True, True, mfma=16, agpr=True, spread=6)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 4, True, True, True, True, mfma=16, early=2, spread=3)),
    # VGPR-staged ring
    (3840, 3840, 128, GemmConfig(128, 128, 64, 64, 64, 1, 2, True, True, False, True)),  # tail
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 128, 2, 1, False, False, False)),
    (512, 1024, 256, GemmConfig(256, 256, 32, 128, 128, 2, 2, True, True, False)),
    (512, 512, 512, GemmConfig(128, 128, 32, 64, 32, 1, 4, True, True, False)),
    (512, 256, 192, GemmConfig(256, 128, 64, 128, 64, 1, 1, True, False, False)),
    (128, 192, 32, GemmConfig(64, 64, 32, 32, 64, 1, 2, False, False, False)),
]

# Full-size shapes: checked on a sample of rows against the CPU checker.
GEMM_FULL = [
    (4096, 4096, 4096, GemmConfig(256, 256, 64, 128, 128, 2, 8, False, True, True)),
    (8192, 8192, 8192, GemmConfig(256, 256, 32, 128, 128, 3, 8, False, True, True)),
    (8192, 8192, 8192, GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True)),
    (6144, 6144, 6144, GemmConfig(256, 256, 64, 128, 64, 2, 8, True, True, True, True)),
    (8192, 8192, 8192, GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=4)),
    (8192, 8192, 8192, GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=4, agpr=True)),
    (8192, 8192, 8192, GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=4, agpr=True, spread=6)),
    (6144, 6144, 6144, GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, True, mfma=16, agpr=True, spread=6)),
]


# bf16 inputs / output (fp32 accumulate)
GEMM_BF16_CASES = [
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, False, False, True)),
    (512, 1024, 256, GemmConfig(128, 128, 32, 64, 64, 3, 2, True, True, True)),
    (256, 256, 192, GemmConfig(64, 64, 64, 32, 32, 1, 1, False, False, False)),
    (3072, 3072, 256, GemmConfig(128, 128, 64, 64, 64, 2, 0, True, True, True, True)),  # block order + tail
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16, early=4)),
    (512, 1024, 256, GemmConfig(128, 128, 32, 64, 64, 3, 2, False, True, True, mfma=16)),
    (512, 512, 512, GemmConfig(256, 256, 64, 128, 64, 2, 1, True, False, True, mfma=16, agpr=True)),
    (512, 1024, 256, GemmConfig(256, 256, 64, 128, 64, 2, 2, True, True, True, mfma=16, early=4, agpr=True, spread=6)),
]


def gemm_specs():
    return ([make_gemm_tc(M, N, K, cfg) for M, N, K, cfg in GEMM_CASES + GEMM_FULL] +
            [make_gemm_tc(M, N, K, cfg, "bfloat16") for M, N, K, cfg in GEMM_BF16_CASES])


# (B, H, S_q, S_kv, D, causal, cfg): sizes the CPU checker finishes in seconds
FA_CASES = [
    (1, 2, 256, 256, 128, False, FAConfig(128, 64, 4, 2)),
    (1, 2, 256, 256, 128, True, FAConfig(128, 64, 4, 2)),
    (2, 2, 512, 512, 64, False, FAConfig(128, 64, 4, 2)),
    (2, 2, 512, 512, 64, True, FAConfig(128, 64, 4, 2)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2)),
    (1, 2, 512, 512, 128, False, FAConfig(256, 32, 8, 1)),
    (1, 1, 256, 256, 128, True, FAConfig(128, 128, 4, 1)),
    (1, 2, 256, 256, 64, True, FAConfig(256, 128, 4, 2)),
    (1, 2, 256, 256, 128, False, FAConfig(128, 32, 2, 2)),
    (1, 3, 128, 640, 128, False, FAConfig(64, 64, 2, 2)),   # S_q != S_kv
    (1, 1, 384, 128, 64, False, FAConfig(128, 128, 4, 1)),
    (1, 1, 128, 128, 128, True, FAConfig(32, 32, 1, 2)),
    (1, 2, 256, 256, 256, False, FAConfig(128, 64, 4, 2)),  # D = 256
    (1, 1, 256, 256, 256, True, FAConfig(64, 32, 2, 2)),
    (2, 4, 512, 512, 64, True, FAConfig(128, 64, 4, 2)),    # causal, whole slices per XCD
    (3, 8, 256, 256, 64, True, FAConfig(64, 64, 2, 2)),
    # S^T computed one tile ahead of the softmax
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, pipe=True)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, pipe=True)),
    (2, 2, 512, 512, 64, True, FAConfig(128, 128, 4, 2, pipe=True)),
    (1, 2, 256, 384, 128, False, FAConfig(128, 128, 4, 2, pipe=True)),
    (1, 1, 128, 64, 64, False, FAConfig(64, 64, 2, 2, pipe=True)),   # a single KV tile
    # slot-interleaved loop: even and odd numbers of KV tiles, one and two query tiles per wave
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, pipe=2)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, pipe=2)),
    (2, 2, 512, 512, 64, True, FAConfig(256, 128, 8, 2, pipe=2)),
    (1, 2, 256, 384, 128, False, FAConfig(128, 128, 4, 2, pipe=2)),  # 3 KV tiles
    (1, 2, 128, 192, 64, False, FAConfig(128, 64, 2, 2, pipe=2)),    # two query tiles per wave
    (1, 1, 128, 64, 64, False, FAConfig(64, 64, 2, 2, pipe=2)),      # a single KV tile
    (1, 1, 128, 128, 64, True, FAConfig(64, 64, 2, 2, pipe=2)),      # two KV tiles, no loop
    # causal slot loop: an odd number of unmasked tiles ahead of the diagonal ones, and
    # key tiles wider than the query tiles
    (1, 2, 512, 512, 64, True, FAConfig(128, 128, 4, 2, pipe=2)),
    (1, 2, 1024, 1024, 64, True, FAConfig(64, 128, 2, 2, pipe=2)),
    # 16x16x32 MFMA tiles (plain loop): full and causal, D = 64 / 128 / 192, one and two LDS
    # stages, one and several query tiles per wave, S_q != S_kv
    (1, 2, 256, 256, 128, False, FAConfig(128, 64, 4, 2, mfma=16)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, mfma=16)),
    (2, 2, 512, 512, 64, True, FAConfig(128, 64, 4, 2, mfma=16)),
    (1, 2, 256, 256, 64, False, FAConfig(256, 128, 4, 2, mfma=16)),
    (1, 3, 128, 640, 128, False, FAConfig(64, 64, 2, 1, mfma=16)),
    (1, 1, 128, 128, 128, True, FAConfig(32, 32, 1, 2, mfma=16)),
    (1, 2, 256, 256, 192, True, FAConfig(128, 64, 4, 2, mfma=16)),
    # ... in the slot loop: full, causal (odd and even numbers of unmasked tiles), D = 64
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, pipe=2, mfma=16)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, pipe=2, mfma=16)),
    (1, 2, 512, 512, 64, True, FAConfig(128, 128, 4, 2, pipe=2, mfma=16)),
    (2, 2, 512, 512, 64, False, FAConfig(128, 64, 4, 2, pipe=2, mfma=16)),
    # head dims that are multiples of 64 but no powers of two: full, causal, the three loops
    (1, 2, 256, 256, 192, False, FAConfig(128, 64, 4, 2)),
    (1, 2, 256, 256, 192, True, FAConfig(128, 64, 4, 2)),
    (1, 2, 256, 384, 192, False, FAConfig(64, 32, 2, 1)),
    (1, 2, 512, 512, 192, True, FAConfig(128, 64, 4, 2, pipe=1)),
    (1, 2, 512, 512, 192, False, FAConfig(128, 64, 4, 2, pipe=2)),
    (1, 2, 512, 512, 192, True, FAConfig(128, 64, 4, 2, pipe=2)),
    (1, 1, 256, 256, 320, True, FAConfig(32, 32, 1, 2)),
    # the plain two-stage loop as one copy of the step (run-time ring slot): both tile
    # forms, full and causal, an odd number of KV tiles
    (1, 2, 512, 512, 128, False, FAConfig(256, 128, 8, 2, mfma=16, roll=True)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 128, 8, 2, roll=True)),
    (2, 2, 256, 320, 64, False, FAConfig(128, 64, 4, 2, roll=True)),
    (1, 2, 512, 512, 64, True, FAConfig(128, 64, 4, 2, mfma=16, roll=True)),
    # Q tile staged in LDS, its fragments read again in every KV step: full and causal,
    # D = 64 / 128 / 192, both tile forms, one to three LDS stages, the three loops, rolled
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, q_in_smem=True)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, q_in_smem=True, mfma=16)),
    (2, 2, 512, 512, 64, False, FAConfig(256, 128, 4, 2, q_in_smem=True, mfma=16)),
    (2, 2, 512, 512, 64, True, FAConfig(128, 64, 4, 2, q_in_smem=True)),
    (1, 2, 256, 256, 192, False, FAConfig(128, 32, 4, 2, q_in_smem=True, mfma=16)),
    (1, 2, 256, 256, 192, True, FAConfig(64, 64, 2, 1, q_in_smem=True)),
    (1, 3, 128, 640, 128, False, FAConfig(64, 64, 2, 1, q_in_smem=True, mfma=16)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, q_in_smem=True, pipe=1)),
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, q_in_smem=True, pipe=2)),
    (2, 2, 512, 512, 64, True, FAConfig(256, 128, 8, 2, q_in_smem=True, pipe=2, mfma=16)),
    (1, 2, 512, 512, 128, True, FAConfig(128, 128, 4, 2, q_in_smem=True, mfma=16, roll=True)),
    (1, 2, 512, 512, 64, False, FAConfig(256, 64, 4, 3, q_in_smem=True, roll=True)),
    # three LDS stages (tiles requested two steps ahead): 1, 2, 4, 5 and 8 KV tiles, full and
    # causal, both tile forms, unrolled by three and rolled
    (1, 2, 128, 64, 64, False, FAConfig(64, 64, 2, 3)),
    (1, 2, 128, 128, 128, True, FAConfig(64, 64, 2, 3, mfma=16)),
    (1, 2, 256, 256, 128, False, FAConfig(128, 64, 4, 3)),
    (1, 2, 256, 320, 64, False, FAConfig(128, 64, 2, 3, mfma=16)),
    (1, 2, 512, 512, 128, True, FAConfig(128, 64, 4, 3)),
    (2, 2, 512, 512, 64, True, FAConfig(256, 64, 4, 3, mfma=16, roll=True)),
    (1, 2, 256, 320, 128, False, FAConfig(128, 64, 4, 3, roll=True)),
    (1, 2, 512, 512, 192, True, FAConfig(128, 32, 4, 3, q_in_smem=True, mfma=16)),
    # the next tile's loads dealt over the first groups of a step: plain and slot loop, both
    # tile forms, full and causal (masked tiles skipped by some waves), odd numbers of tiles
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, pipe=2, spread=8)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, pipe=2, mfma=16, spread=4)),
    (2, 2, 512, 512, 64, True, FAConfig(256, 128, 8, 2, pipe=2, spread=8)),
    (1, 2, 256, 384, 128, False, FAConfig(128, 128, 4, 2, pipe=2, spread=100)),
    (2, 2, 512, 512, 64, False, FAConfig(256, 64, 4, 2, spread=4)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, mfma=16, spread=2)),
    (1, 2, 256, 320, 64, False, FAConfig(128, 64, 4, 2, spread=1)),
    (1, 2, 512, 512, 64, True, FAConfig(128, 128, 4, 2, q_in_smem=True, spread=4)),
    (2, 2, 512, 512, 64, False, FAConfig(256, 64, 4, 3, spread=4)),
    (1, 2, 512, 512, 128, True, FAConfig(128, 64, 4, 3, mfma=16, spread=2)),
    (1, 2, 256, 320, 64, False, FAConfig(128, 64, 2, 3, spread=100)),
    # exponentials against the running max as it stands (`trust`): both tile forms, two and
    # three stages, unrolled and rolled, with the load window and the staged Q tile, full and
    # causal (tiles that reach the diagonal always take their max), D = 64 / 128 / 192,
    # one, two and an odd number of tiles
    (1, 2, 512, 512, 128, False, FAConfig(256, 128, 8, 2, mfma=16, roll=True, trust=True)),
    (2, 2, 512, 512, 64, False, FAConfig(256, 64, 4, 3, trust=True)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 128, 8, 2, mfma=16, roll=True, trust=True)),
    (2, 2, 512, 512, 64, True, FAConfig(256, 64, 4, 3, trust=True)),
    (1, 2, 256, 320, 64, False, FAConfig(128, 64, 4, 2, trust=True)),
    (1, 2, 256, 320, 128, False, FAConfig(128, 64, 4, 2, mfma=16, spread=4, trust=True)),
    (1, 2, 512, 512, 128, True, FAConfig(256, 64, 8, 2, spread=4, trust=True)),
    (1, 2, 256, 256, 192, False, FAConfig(128, 32, 4, 2, q_in_smem=True, mfma=16, trust=True)),
    (1, 2, 256, 256, 192, True, FAConfig(128, 32, 4, 3, q_in_smem=True, trust=True)),
    (1, 2, 128, 64, 64, False, FAConfig(64, 64, 2, 3, trust=True)),
    (1, 2, 128, 128, 128, True, FAConfig(64, 64, 2, 2, mfma=16, roll=True, trust=True)),
    (1, 3, 128, 640, 128, False, FAConfig(64, 64, 2, 3, roll=True, trust=True)),
    # linear LDS rows (no swizzle): both row lengths, both tile forms, with and without the
    # staged Q tile
    (1, 2, 256, 256, 128, True, FAConfig(128, 64, 4, 2, swizzle=False)),
    (1, 2, 256, 256, 64, False, FAConfig(128, 64, 4, 2, swizzle=False, mfma=16)),
    (1, 2, 256, 256, 64, True, FAConfig(128, 64, 4, 1, q_in_smem=True, swizzle=False)),
    (1, 2, 512, 512, 128, False, FAConfig(256, 64, 8, 2, q_in_smem=True, swizzle=False, pipe=2, mfma=16)),
]

FA_FULL = [
    (4, 16, 4096, 4096, 128, False, FAConfig(128, 64, 4, 2)),
    (4, 16, 4096, 4096, 128, True, FAConfig(128, 64, 4, 2)),
    (4, 16, 4096, 4096, 64, False, FAConfig(128, 64, 4, 2)),
    (4, 16, 4096, 4096, 64, True, FAConfig(128, 64, 4, 2)),
    (4, 16, 4096, 4096, 128, True, FAConfig(256, 128, 8, 2)),
    (4, 16, 4096, 4096, 64, False, FAConfig(256, 128, 8, 2, pipe=2)),
    (4, 16, 4096, 4096, 128, False, FAConfig(256, 64, 8, 2, pipe=2)),
    (4, 16, 4096, 4096, 128, True, FAConfig(256, 64, 8, 2, pipe=2)),
    (4, 16, 4096, 4096, 128, False, FAConfig(256, 64, 8, 2, q_in_smem=True, mfma=16)),
    (4, 16, 4096, 4096, 64, True, FAConfig(256, 64, 4, 3, q_in_smem=True)),
    (4, 16, 4096, 4096, 128, True, FAConfig(256, 64, 8, 2, pipe=2, spread=8)),
    (4, 16, 4096, 4096, 64, False, FAConfig(256, 64, 4, 2, spread=4)),
    (4, 16, 4096, 4096, 128, False, FAConfig(256, 128, 8, 2, mfma=16, roll=True, trust=True)),
    (4, 16, 4096, 4096, 64, False, FAConfig(256, 64, 4, 3, trust=True)),
    (4, 16, 4096, 4096, 64, True, FAConfig(256, 64, 4, 2, spread=4, trust=True)),
]


def fa_specs():
    return [make_flash_attn_fwd(B, H, Sq, Skv, D, cfg, None, causal)
            for B, H, Sq, Skv, D, causal, cfg in FA_CASES + FA_FULL]


def spilling_specs():
    """The same code object twice: an attention kernel at D = 320 whose registers do not fit
    (80 bytes of scratch per lane), plain and marked as one that must not spill.  The kernel
    only ever waits with vmcnt(0), so it is correct as it is; the mark is what the loader's
    refusal is tested with."""
    from deca_amd.kernels.build import make_spec

    plain = make_flash_attn_fwd(1, 2, 256, 256, 320, FAConfig(128, 64, 4, 2), None, False)
    marked = make_spec(plain.template, dict(plain.defines), plain.grid, plain.block, plain.nargs,
                       lds_bytes=plain.lds_bytes, options=list(plain.options),
                       meta=dict(dict(plain.meta), no_scratch=True))
    return plain, marked


# Shapes whose solver output runs on the GPU config by config (test_all_configs_gpu.py):
# a sample of SAMPLE evenly spaced configurations each by default.
SOLVER_FA_SHAPES = [(2, 16, 1024, 64, False), (2, 16, 1024, 64, True), (2, 16, 1024, 128, False),
                    (2, 16, 1024, 128, True), (1, 16, 2048, 256, True), (2, 16, 1024, 192, False),
                    (2, 16, 1024, 192, True)]
SOLVER_GEMM_SHAPES = [(2048, 2048, 2048), (3072, 3072, 512)]  # the second leaves partial waves (tail)
SOLVER_ROW_SHAPES = [("softmax", 2048, 4096, "float16"), ("rmsnorm", 2048, 8192, "bfloat16"),
                     ("softmax", 512, 32000, "float16"), ("rmsnorm", 512, 128256, "float16")]
SAMPLE = 24


def solver_sample(configs, n: int = SAMPLE):
    """`n` evenly spaced entries of a solver's list (all of it when it is shorter)."""
    if len(configs) <= n:
        return list(configs)
    return [configs[(i * len(configs)) // n] for i in range(n)]


def solver_sample_specs():
    from deca_amd import Solver
    from deca_amd.arch.MI355X import MI355X

    arch = MI355X()
    specs = []
    for B, H, S, D, causal in SOLVER_FA_SHAPES:
        specs += [make_flash_attn_fwd(B, H, S, S, D, cfg, None, causal)
                  for cfg in solver_sample(Solver.solve_flash_attn(arch, B, H, S, S, D))]
    for M, N, K in SOLVER_GEMM_SHAPES:
        specs += [make_gemm_tc(M, N, K, cfg) for cfg in solver_sample(Solver.solve_gemm_tc(arch, M, N, K))]
    for op, M, N, dtype in SOLVER_ROW_SHAPES:
        specs += [make_rowwise(op, M, N, dtype, cfg, 1e-6)
                  for cfg in solver_sample(Solver.solve_rowwise(arch, op, M, N))]
    return specs


def all_specs():
    return (rowwise_specs() + gemm_specs() + fa_specs() + [spilling_specs()[0]]
            + solver_sample_specs())
