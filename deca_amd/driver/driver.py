"""
ctypes binding of libdeca_hip.so plus the CU occupancy calculator.

The reference's src/driver/driver.py simulates CUDA occupancy and the
shared-memory carve-out (:11-47, :98-202); CDNA has no carve-out, so the
occupancy part is `cu_occupancy` (waves per SIMD from VGPRs and LDS).  The
binding replaces `tvm.runtime.load_module(path)["main"]`
(src/RuntimeMod.py:104-109, :204-208).
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char, c_char_p, c_float, c_int, c_size_t, c_uint, c_void_p

from deca_amd.driver.build_lib import LIB_PATH


class DevInfo(ctypes.Structure):
    _fields_ = [
        ("name", c_char * 256),
        ("gcn_arch", c_char * 256),
        ("cu_count", c_int),
        ("clock_khz", c_int),
        ("mem_clock_khz", c_int),
        ("mem_bus_bits", c_int),
        ("wave_size", c_int),
        ("l2_bytes", c_int),
        ("max_threads_per_block", c_int),
        ("max_threads_per_cu", c_int),
        ("regs_per_block", c_int),
        ("reserved", c_int),
        ("lds_per_block", c_size_t),
        ("lds_per_cu", c_size_t),
        ("total_mem", c_size_t),
    ]


class FuncInfo(ctypes.Structure):
    _fields_ = [
        ("num_regs", c_int),
        ("static_lds_bytes", c_int),
        ("scratch_bytes", c_int),
        ("max_threads_per_block", c_int),
        ("const_bytes", c_int),
        ("reserved", c_int),
    ]


# name -> (restype, argtypes); also the list the symbol-export test checks.
C_API = {
    "deca_init": (c_int, [c_int]),
    "deca_device_count": (c_int, [POINTER(c_int)]),
    "deca_device_info": (c_int, [c_int, POINTER(DevInfo)]),
    "deca_module_load": (c_int, [c_char_p, POINTER(c_void_p)]),
    "deca_module_load_data": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "deca_module_unload": (c_int, [c_void_p]),
    "deca_get_function": (c_int, [c_void_p, c_char_p, POINTER(c_void_p)]),
    "deca_function_info": (c_int, [c_void_p, POINTER(FuncInfo)]),
    "deca_set_max_dynamic_lds": (c_int, [c_void_p, c_uint]),
    "deca_launch": (c_int, [c_void_p] + [c_uint] * 7 + [c_void_p, POINTER(c_void_p), c_uint]),
    "deca_launch_timed": (
        c_int,
        [c_void_p] + [c_uint] * 7 + [c_void_p, POINTER(c_void_p), c_uint, c_uint, c_uint,
                                     POINTER(c_float)],
    ),
    "deca_launch_between": (
        c_int,
        [c_void_p] + [c_uint] * 7 + [c_void_p, POINTER(c_void_p), c_uint, c_uint, c_uint,
                                     c_void_p, c_void_p],
    ),
    "deca_synchronize": (c_int, [c_void_p]),
    "deca_error_string": (c_char_p, [c_int]),
}


class DeviceInfo:
    """Plain-Python copy of `deca_devinfo`."""

    def __init__(self, raw: DevInfo):
        self.name = raw.name.decode(errors="replace")
        self.gcn_arch = raw.gcn_arch.decode(errors="replace")
        for f, _ in DevInfo._fields_[2:]:
            setattr(self, f, int(getattr(raw, f)))

    def __repr__(self):
        return f"DeviceInfo({self.__dict__})"


class HipDriver:
    """Thin wrapper over the C ABI; raises RuntimeError on any non-zero code."""

    def __init__(self, lib_path: str = LIB_PATH):
        if not os.path.exists(lib_path):
            raise RuntimeError(
                f"{lib_path} is missing: build it with `python -m deca_amd.driver.build_lib` "
                "(there is no fallback path without the HIP launcher library)"
            )
        # torch ships its own copy of the HIP runtime under the same soname
        # (libamdhip64.so.7).  Tensors come from torch, so its runtime must be the
        # one in the process: import it before this library is mapped, otherwise
        # the system copy is loaded first and torch later finds "no ROCm-capable
        # device".
        try:
            import torch  # noqa: F401
        except ImportError:  # the library also works standalone (raw device pointers)
            pass
        self.lib = ctypes.CDLL(lib_path)
        for name, (restype, argtypes) in C_API.items():
            fn = getattr(self.lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        self._initialised = set()

    def check(self, code: int, what: str = ""):
        if code != 0:
            msg = self.lib.deca_error_string(code).decode(errors="replace")
            raise RuntimeError(f"{what or 'HIP call'} failed: {msg} (hipError {code})")

    def init(self, dev: int = 0):
        if dev not in self._initialised:
            self.check(self.lib.deca_init(dev), f"deca_init({dev})")
            self._initialised.add(dev)

    def device_count(self) -> int:
        n = c_int(0)
        self.check(self.lib.deca_device_count(byref(n)), "deca_device_count")
        return n.value

    def device_info(self, dev: int = 0) -> DeviceInfo:
        raw = DevInfo()
        self.check(self.lib.deca_device_info(dev, byref(raw)), "deca_device_info")
        return DeviceInfo(raw)

    def module_load(self, path: str) -> c_void_p:
        mod = c_void_p()
        self.check(self.lib.deca_module_load(path.encode(), byref(mod)), f"deca_module_load({path})")
        return mod

    def module_unload(self, mod: c_void_p):
        self.check(self.lib.deca_module_unload(mod), "deca_module_unload")

    def get_function(self, mod: c_void_p, sym: str) -> c_void_p:
        fn = c_void_p()
        self.check(self.lib.deca_get_function(mod, sym.encode(), byref(fn)), f"deca_get_function({sym})")
        return fn

    def function_info(self, fn: c_void_p) -> dict:
        raw = FuncInfo()
        self.check(self.lib.deca_function_info(fn, byref(raw)), "deca_function_info")
        return {f: int(getattr(raw, f)) for f, _ in FuncInfo._fields_ if f != "reserved"}

    def set_max_dynamic_lds(self, fn: c_void_p, nbytes: int):
        self.check(self.lib.deca_set_max_dynamic_lds(fn, nbytes), "deca_set_max_dynamic_lds")

    def launch(self, fn, grid, block, lds_bytes, stream, ptrs):
        n = len(ptrs)
        arr = (c_void_p * n)(*ptrs)
        self.check(
            self.lib.deca_launch(fn, *grid, *block, lds_bytes, c_void_p(stream), arr, n),
            "deca_launch",
        )

    @staticmethod
    def pack_sets(ptr_sets):
        """(array of all pointers, pointers per set, number of sets) of a list of equally
        long pointer tuples, in the layout `deca_launch_timed` / `deca_launch_between` read."""
        nsets, n = len(ptr_sets), len(ptr_sets[0])
        flat = [p for s in ptr_sets for p in s]
        return (c_void_p * (nsets * n))(*flat), n, nsets

    def launch_timed(self, fn, grid, block, lds_bytes, stream, ptr_sets, iters) -> float:
        """Seconds per launch, averaged over `iters` back-to-back launches that
        cycle through `ptr_sets` (a list of equally long pointer tuples)."""
        arr, n, nsets = self.pack_sets(ptr_sets)
        ms = c_float(0.0)
        self.check(
            self.lib.deca_launch_timed(
                fn, *grid, *block, lds_bytes, c_void_p(stream), arr, n, nsets, iters, byref(ms)
            ),
            "deca_launch_timed",
        )
        return ms.value / 1e3 / iters

    def batch_call(self, fn, grid, block, lds_bytes, stream, packed, iters,
                   start_event: int = 0, stop_event: int = 0):
        """A callable without arguments that enqueues `iters` back-to-back launches cycling
        through `packed` (from `pack_sets`) and returns without waiting.  `start_event` /
        `stop_event` are hipEvent_t handles of the caller (0: none), recorded on the stream
        directly before the first and after the last launch.  Every argument is converted
        here, so that the call itself is one foreign-function call."""
        arr, n, nsets = packed
        cargs = ([fn] + [c_uint(v) for v in (*grid, *block, lds_bytes)]
                 + [c_void_p(stream), arr, c_uint(n), c_uint(nsets), c_uint(iters),
                    c_void_p(start_event or None), c_void_p(stop_event or None)])
        entry, check = self.lib.deca_launch_between, self.check

        def call():
            check(entry(*cargs), "deca_launch_between")

        return call

    def synchronize(self, stream: int = 0):
        self.check(self.lib.deca_synchronize(c_void_p(stream)), "deca_synchronize")


_driver: HipDriver | None = None


def get_driver() -> HipDriver:
    global _driver
    if _driver is None:
        _driver = HipDriver()
    return _driver


class KernelRejected(RuntimeError):
    """A code object that loads but must not be launched (see LoadedKernel)."""


class LoadedKernel:
    """A code object loaded on the device plus its launch geometry.

    Calling it with torch tensors (in the operator's `kernel_args` order)
    launches `deca_main` on torch's current stream, like the PackedFunc the
    reference gets from `load_module(path)["main"]`.
    """

    def __init__(self, spec, path: str, device: int = 0):
        self.spec = spec
        self.path = path
        self.launches = 0  # launches issued through this object so far
        self.drv = get_driver()
        self.drv.init(device)
        self.mod = self.drv.module_load(path)
        self.fn = self.drv.get_function(self.mod, spec.symbol)
        if spec.lds_bytes > 64 * 1024:
            self.drv.set_max_dynamic_lds(self.fn, spec.lds_bytes)
        # A kernel whose loop waits for "all but the newest n" of its global->LDS loads
        # (s_waitcnt vmcnt(n), n > 0) counts on those loads being the loop's only vector
        # memory traffic.  Register spills put scratch stores into the same counter, and
        # stores retire out of order with respect to loads: the wait may then pass with a
        # tile still in flight.  Such a code object is refused instead of launched.
        meta = dict(spec.meta)
        if meta.get("no_scratch"):
            scratch = self.info()["scratch_bytes"]
            if scratch > 0:
                self.close()
                raise KernelRejected(
                    f"{spec.template} [{meta.get('cfg', '')}] spills {scratch} bytes per lane to "
                    "scratch memory; its partial vmcnt waits are only valid without spills")

    def info(self) -> dict:
        return self.drv.function_info(self.fn)

    @staticmethod
    def _stream() -> int:
        import torch

        return int(torch.cuda.current_stream().cuda_stream)

    def _ptrs(self, tensors):
        if len(tensors) != self.spec.nargs:
            raise ValueError(f"kernel takes {self.spec.nargs} tensors, got {len(tensors)}")
        for t in tensors:
            if not (t.is_cuda and t.is_contiguous()):
                raise ValueError("kernel arguments must be contiguous device tensors")
        return [t.data_ptr() for t in tensors]

    def __call__(self, *tensors):
        self.launches += 1
        self.drv.launch(
            self.fn, self.spec.grid, self.spec.block, self.spec.lds_bytes, self._stream(),
            self._ptrs(tensors),
        )

    def time(self, tensor_sets, iters: int) -> float:
        """Average seconds per launch over `iters` back-to-back launches cycling
        through `tensor_sets` (list of argument tuples)."""
        self.launches += iters
        return self.drv.launch_timed(
            self.fn, self.spec.grid, self.spec.block, self.spec.lds_bytes, self._stream(),
            [self._ptrs(ts) for ts in tensor_sets], iters,
        )

    def pack(self, tensor_sets):
        """The argument sets in the form `batch` takes (built once, outside a timed region);
        the tensors must stay alive while it is in use."""
        return self.drv.pack_sets([self._ptrs(ts) for ts in tensor_sets])

    def batch_call(self, packed, iters: int, start=None, stop=None):
        """A callable without arguments that enqueues `iters` back-to-back launches cycling
        through the packed argument sets on the stream that is current now, and does not
        wait.  `start` / `stop`: torch.cuda.Event objects that have been recorded before (an
        event is created at its first record), recorded again directly before the first and
        after the last launch.  Prepared outside a timed region, called inside it."""
        run = self.drv.batch_call(
            self.fn, self.spec.grid, self.spec.block, self.spec.lds_bytes, self._stream(), packed, iters,
            0 if start is None else int(start.cuda_event), 0 if stop is None else int(stop.cuda_event),
        )

        def call():
            self.launches += iters
            run()

        return call

    def batch(self, packed, iters: int, start=None, stop=None) -> None:
        """`batch_call(...)()`."""
        self.batch_call(packed, iters, start, stop)()

    def close(self):
        if getattr(self, "mod", None) is not None and self.mod:
            try:
                self.drv.module_unload(self.mod)
            finally:
                self.mod = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001  (interpreter shutdown)
            pass


def load_kernel(spec, path: str, device: int = 0) -> LoadedKernel:
    return LoadedKernel(spec, path, device)


# ---------------------------------------------------------------------------
# occupancy
# ---------------------------------------------------------------------------
def cu_occupancy(arch, vgprs: int, lds_bytes: int, threads: int) -> tuple[int, int]:
    """Returns (resident workgroups per CU, waves per SIMD) of a kernel using
    `vgprs` unified registers per lane (arch + accumulation), `lds_bytes` of LDS
    per workgroup and `threads` work-items.

    CDNA rules: each SIMD has a 512-entry unified VGPR file per lane allocated
    in `vgpr_granule` blocks, at most `max_waves_per_simd` waves per SIMD, LDS
    shared by the workgroups of a CU, and a workgroup's waves are spread over
    the CU's SIMDs.
    """
    waves = -(-threads // arch.warp_size)
    gran = arch.vgpr_granule
    regs = max(gran, -(-max(vgprs, 1) // gran) * gran)
    waves_by_regs = min(arch.max_waves_per_simd, arch.vgprs_per_simd // regs)
    if waves_by_regs == 0:
        return 0, 0
    simds = arch.simds_per_cu
    # A workgroup puts ceil(waves / simds) waves on its busiest SIMD.
    per_simd = -(-waves // simds)
    wgs_by_regs = (waves_by_regs // per_simd) if waves >= simds else (waves_by_regs * simds) // waves
    wgs_by_lds = arch.lds_per_cu // lds_bytes if lds_bytes > 0 else 1 << 30
    wgs_by_waves = (arch.max_waves_per_simd * simds) // waves
    wgs = max(0, min(wgs_by_regs, wgs_by_lds, wgs_by_waves, arch.max_resident_blocks_per_sm))
    return int(wgs), int(min(arch.max_waves_per_simd, -(-wgs * waves // simds)))
