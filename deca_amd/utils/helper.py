"""GPU detection and small helpers (reference: src/utils/helper.py:19-25, :50-99)."""

from __future__ import annotations

from deca_amd.arch.MI355X import MI355X


def byte_size(dtype: str) -> int:
    sizes = {"float32": 4, "float16": 2, "bfloat16": 2}
    if dtype not in sizes:
        raise ValueError(f"Unsupported data type: {dtype}")
    return sizes[dtype]


class GPUDetector:
    """Maps the visible device to its hardware model.

    The reference keys on the device name (helper.py:54-63).  ROCm reports
    marketing names inconsistently ("AMD Instinct MI355X", "AMD Radeon
    Graphics" when the id table is missing), so the offload architecture is the
    primary key and the name a secondary one.
    """

    GPU_ARCH_MAP = {"gfx950": MI355X}
    GPU_MODEL_MAP = {"AMD Instinct MI355X": MI355X, "AMD Instinct MI350X": MI355X}

    @classmethod
    def _device_info(cls, device_id: int = 0):
        from deca_amd.driver.driver import get_driver

        drv = get_driver()
        if drv.device_count() <= device_id:
            raise RuntimeError("no HIP device is visible")
        drv.init(device_id)
        return drv.device_info(device_id)

    @classmethod
    def lookup(cls, name: str, gcn_arch: str):
        """Pure mapping step (host only, testable without a device)."""
        arch = gcn_arch.split(":")[0]
        if arch in cls.GPU_ARCH_MAP:
            return cls.GPU_ARCH_MAP[arch]
        if name in cls.GPU_MODEL_MAP:
            return cls.GPU_MODEL_MAP[name]
        raise NotImplementedError(
            f"Unsupported GPU: {name} ({gcn_arch}); supported architectures: "
            f"{sorted(cls.GPU_ARCH_MAP)}, names: {sorted(cls.GPU_MODEL_MAP)}"
        )

    @classmethod
    def detect_gpu(cls, verbose: bool, device_id: int = 0):
        """Detect the current GPU model; prints and exits on failure like the
        reference (helper.py:87-89)."""
        try:
            info = cls._device_info(device_id)
            if verbose:
                print(f"Detected GPU: {info.name} ({info.gcn_arch})")
            return cls.lookup(info.name, info.gcn_arch)
        except Exception as e:  # noqa: BLE001
            print(f"GPU detection failed: {e}")
            raise SystemExit(-1)

    @classmethod
    def create_gpu_instance(cls, verbose=True, device_id: int = 0):
        gpu_class = cls.detect_gpu(verbose=verbose, device_id=device_id)
        gpu = gpu_class()
        if hasattr(gpu, "configure_device"):
            gpu.configure_device(cls._device_info(device_id))
        return gpu
