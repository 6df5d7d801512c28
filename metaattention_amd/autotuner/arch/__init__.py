"""Device descriptors.  The reference keys its tile search on these
(attention_engine/autotuner/arch/__init__.py:19-34); this package has fixed
CDNA4 tile tables instead, so the descriptor only documents the machine and
provides ``.name`` for user scripts that build tuning-file paths with it."""


class Arch:
    name = "base"
    platform = "unknown"


class MI355X(Arch):
    def __init__(self):
        self.name = "MI355X"
        self.platform = "ROCM"
        self.compute_capability = "gfx950"
        self.compute_max_core = 256          # CUs
        self.xcds = 8
        self.warp_size = 64
        self.simd_per_cu = 4
        self.smem_cap = 160 * 1024           # LDS bytes per CU
        self.vgpr_per_simd_lane = 512        # unified arch + accumulation VGPRs
        self.mma_primitive = [32, 32, 16]    # v_mfma_f32_32x32x16_bf16
        self.peak_bf16_tflops = 2500.0
        self.hbm_bandwidth_gbs = 8000.0
        self.hbm_bytes = 288 * 2**30
        self.l2_bytes_per_xcd = 4 * 2**20
        self.transaction_size = [64, 128]


def get_attn_device():
    """Always MI355X: the kernel library has no other target."""
    return MI355X()
