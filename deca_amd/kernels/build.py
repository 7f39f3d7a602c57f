"""
Shared compilation helpers for the hand-written HIP kernel templates.

Counterpart of the reference's src/kernels/build.py (nvcc callback :56-64,
`build_kernel` :73-87, `cuda_target` :67-70): a kernel is a `.hip` template
under `deca_amd/csrc/` specialised with `-D` macros and compiled by
`hipcc --genco` into a gfx950 code object.  Nothing here imports torch or
touches the GPU, so it is safe inside spawned compile workers.
"""

from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import tempfile
import threading
from dataclasses import dataclass, field

PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(PKG_ROOT, "csrc")
CACHE_DIR = os.path.join(PKG_ROOT, "_kcache")
KERNEL_SYMBOL = "deca_main"
DEFAULT_ARCH = "gfx950"

# The reference passes --use_fast_math to nvcc (build.py:9).
FAST_MATH_OPTIONS = ["-ffast-math"]
# Packed-FP32 VALU forms are switched off for every device compile.
BASE_OPTIONS = ["-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


@dataclass(frozen=True)
class KernelSpec:
    """Everything needed to compile and launch one specialised kernel.

    Plays the role of the IRModule returned by the reference's `make_*`
    functions: the template plus its compile-time constants, and the launch
    geometry the reference derives in gemm_tir.py:156, rowwise_tir.py:128 and
    flash_attn_tir.py:147.
    """

    template: str  # file name under csrc/
    defines: tuple  # ((name, value), ...) sorted
    grid: tuple  # (gx, gy, gz)
    block: tuple  # (bx, by, bz)
    nargs: int  # device pointers the kernel takes
    lds_bytes: int = 0  # dynamic LDS (static LDS lives in the code object)
    options: tuple = tuple(FAST_MATH_OPTIONS)
    symbol: str = KERNEL_SYMBOL
    meta: tuple = field(default=(), compare=False)  # free-form (name, value) notes

    @property
    def source_path(self) -> str:
        return os.path.join(CSRC_DIR, self.template)

    def define_flags(self) -> list[str]:
        return [f"-D{k}={v}" for k, v in self.defines]

    def key(self) -> str:
        """Content hash: template text (with the csrc files it includes) + macros + options."""
        h = hashlib.sha1()
        with open(self.source_path, "rb") as f:
            text = f.read()
        h.update(text)
        # files of csrc/ that the template includes are part of the kernel's source
        for name in re.findall(rb'^#include "([^"]+)"', text, re.M):
            inc = os.path.join(CSRC_DIR, name.decode())
            if os.path.exists(inc):
                with open(inc, "rb") as f:
                    h.update(f.read())
        h.update(repr((self.defines, self.options, BASE_OPTIONS)).encode())
        return h.hexdigest()[:20]

    def show(self) -> str:
        defs = " ".join(self.define_flags())
        return f"{self.template} grid={self.grid} block={self.block} lds={self.lds_bytes}\n  {defs}"


def make_spec(template, defines: dict, grid, block, nargs, lds_bytes=0, options=None, meta=None):
    def norm(v):
        if isinstance(v, bool):
            return int(v)
        return v

    return KernelSpec(
        template=template,
        defines=tuple(sorted((k, norm(v)) for k, v in defines.items())),
        grid=tuple(int(g) for g in grid),
        block=tuple(int(b) for b in block),
        nargs=int(nargs),
        lds_bytes=int(lds_bytes),
        options=tuple(FAST_MATH_OPTIONS if options is None else options),
        meta=tuple(sorted((meta or {}).items())),
    )


def rocm_target(device_id: int = 0) -> str:
    """Offload architecture of the visible device (reference: `cuda_target`, build.py:67-70)."""
    from deca_amd.driver.driver import get_driver

    arch = get_driver().device_info(device_id).gcn_arch
    return arch.split(":")[0] or DEFAULT_ARCH


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def compile_command(spec: KernelSpec, arch: str, out_path: str) -> list[str]:
    return [
        hipcc_path(), "--genco", f"--offload-arch={arch}", *BASE_OPTIONS, *spec.options,
        *spec.define_flags(), spec.source_path, "-o", out_path,
    ]


def check_generated_code(spec: KernelSpec, asm_text: str) -> None:
    """What a spec promises about its generated ISA (`meta`), checked on the assembly text.

    `accumulator_moves`: the kernel keeps MFMA accumulators in accumulation registers through
    inline assembly, with the wait states around them placed by hand.  That is only valid
    while the compiler never touches an accumulator between its initialisation and the
    epilogue, so the number of `v_accvgpr_*` instructions must be exactly the promised one
    and nothing may spill."""
    meta = dict(spec.meta)
    want = meta.get("accumulator_moves")
    if want is None:
        return
    got = len(re.findall(r"^\s*v_accvgpr_(?:read|write|mov)_b32", asm_text, re.M))
    spills = [int(v) for v in re.findall(r"\.vgpr_spill_count:\s*(\d+)", asm_text)]
    scratch = [int(v) for v in re.findall(r"\.private_segment_fixed_size:\s*(\d+)", asm_text)]
    if got != want or any(spills) or any(scratch):
        raise RuntimeError(
            f"{spec.template} [{meta.get('cfg', '')}]: {got} accumulation-register moves where "
            f"{want} are accounted for, {sum(spills)} spilled registers: the compiler moves "
            "accumulators it cannot know to be in flight")
    late = late_operand_writes(asm_text)
    if late:
        raise RuntimeError(
            f"{spec.template} [{meta.get('cfg', '')}]: accumulation-register moves aside, a vector "
            f"instruction writes an MFMA operand less than two wait states before it: {late[0]}")


def _vgprs(operand: str) -> set:
    """Vector registers named by one assembly operand: v7, v[4:7]; anything else: none."""
    m = re.fullmatch(r"v(\d+)", operand)
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    return set(range(int(m.group(1)), int(m.group(2)) + 1)) if m else set()


def late_operand_writes(asm_text: str) -> list:
    """MFMAs with accumulation-register results (the hand-written ones) whose A or B operand
    is written by a vector-ALU instruction fewer than two wait states earlier, in program
    text order: every instruction between counts one state, `s_nop n` counts n + 1.  The
    hardware needs two; the compiler provides them for MFMAs it knows, not behind inline
    assembly.  Returns descriptions of the offending pairs."""
    bad, recent = [], []  # recent: (states this instruction adds, registers it writes, text)
    for raw in asm_text.splitlines():
        line = raw.split(";")[0].strip()
        if not line or line.startswith(".") or line.endswith(":"):
            continue
        op, _, rest = line.partition(" ")
        args = [a.strip() for a in rest.split(",")] if rest else []
        if op.startswith("v_mfma") and args and args[0].startswith("a"):
            reads = _vgprs(args[1]) | _vgprs(args[2]) if len(args) > 2 else set()
            states = 0
            for adds, writes, text in reversed(recent):
                if states >= 2:
                    break
                if writes & reads:
                    bad.append(f"`{text}` before `{line}`")
                    break
                states += adds
        if op == "s_nop":
            recent.append((int(args[0]) + 1 if args else 1, set(), line))
        elif op.startswith("v_") and not op.startswith("v_mfma") and not op.startswith("v_cmp"):
            recent.append((1, _vgprs(args[0]) if args else set(), line))
        else:
            recent.append((1, set(), line))
        del recent[:-4]
    return bad


# The checks of `check_generated_code` read compiler output as text: which instructions the
# register allocator adds and where the scheduler puts them is a property of one compiler.
# They were validated (every `agpr=1` configuration of two shapes built, checked and run
# against torch on the GPU) with this hipcc; under another one a kernel that relies on them
# is refused unless DECA_ALLOW_UNCHECKED_HIPCC=1.
VALIDATED_HIPCC = "HIP version: 7.2.26015"
_hipcc_version = None


def hipcc_version() -> str:
    """First line of `hipcc --version` (cached)."""
    global _hipcc_version
    if _hipcc_version is None:
        proc = subprocess.run([hipcc_path(), "--version"], capture_output=True, text=True)
        _hipcc_version = (proc.stdout.splitlines() or [""])[0].strip()
    return _hipcc_version


def require_validated_hipcc(spec: KernelSpec) -> None:
    if os.environ.get("DECA_ALLOW_UNCHECKED_HIPCC") == "1":
        return
    have = hipcc_version()
    if not have.startswith(VALIDATED_HIPCC):
        raise RuntimeError(
            f"{spec.template} [{dict(spec.meta).get('cfg', '')}] relies on checks of the generated "
            f"code that were validated with '{VALIDATED_HIPCC}...'; this is '{have}'. Set "
            "DECA_ALLOW_UNCHECKED_HIPCC=1 to build it anyway.")


def build_kernel(spec: KernelSpec, arch: str | None, path: str, dump_dir: str | None = None) -> str:
    """Compiles `spec` into the code object `path`; `dump_dir` keeps the
    generated ISA for inspection, as `<template>_<key>.s` (reference: build.py:73-87).  A
    spec that makes promises about its generated code (`check_generated_code`) is compiled
    with the ISA kept and refused when they do not hold.  The compiler's intermediate
    files go to a directory of this build's own, so that neither another build's
    assembly nor a stale file can be the one that is checked or kept."""
    arch = arch or DEFAULT_ARCH
    os.makedirs(os.path.dirname(os.path.abspath(path)) or ".", exist_ok=True)
    tmp = f"{path}.tmp{os.getpid()}_{threading.get_ident()}"
    cmd = compile_command(spec, arch, tmp)
    checked = "accumulator_moves" in dict(spec.meta)
    if checked:
        require_validated_hipcc(spec)
    work_dir = tempfile.mkdtemp(prefix="deca_isa_") if (checked or dump_dir) else None
    if work_dir:
        cmd.append("--save-temps")
    try:
        proc = subprocess.run(cmd, capture_output=True, text=True, cwd=work_dir)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {spec.show()}:\n{proc.stderr[-4000:]}")
        if work_dir:
            stem = os.path.splitext(spec.template)[0]
            kept = [f for f in os.listdir(work_dir)
                    if f.endswith(".s") and "amdgcn" in f and f.startswith(stem + "-")]
            if len(kept) != 1:
                raise RuntimeError(f"expected one device assembly file for {spec.show()}, found {kept}")
            asm_path = os.path.join(work_dir, kept[0])
            if checked:
                with open(asm_path) as f:
                    check_generated_code(spec, f.read())
            if dump_dir:
                os.makedirs(dump_dir, exist_ok=True)
                shutil.copyfile(asm_path, os.path.join(dump_dir, f"{stem}_{spec.key()}.s"))
    except Exception:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise
    finally:
        if work_dir:
            shutil.rmtree(work_dir, ignore_errors=True)
    os.replace(tmp, path)
    return path


def cached_build(spec: KernelSpec, arch: str | None = None) -> str:
    """Path of the code object of `spec` in the in-tree cache, compiling on a miss."""
    arch = arch or DEFAULT_ARCH
    path = os.path.join(CACHE_DIR, f"{os.path.splitext(spec.template)[0]}_{arch}_{spec.key()}.hsaco")
    if not os.path.exists(path):
        build_kernel(spec, arch, path)
    return path


def kernel_resources(spec: KernelSpec, arch: str | None = None) -> dict:
    """Compiles `spec` to assembly and returns the resource usage the code
    object records (VGPRs, AGPRs, SGPRs, LDS, spills).  Host only."""
    arch = arch or DEFAULT_ARCH
    with tempfile.TemporaryDirectory(prefix="deca_res_") as d:
        asm = os.path.join(d, "k.s")
        cmd = [
            hipcc_path(), "-S", "--cuda-device-only", f"--offload-arch={arch}", *BASE_OPTIONS,
            *spec.options, *spec.define_flags(), spec.source_path, "-o", asm,
        ]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {spec.show()}:\n{proc.stderr[-4000:]}")
        out = {}
        keys = {
            ".vgpr_count:": "vgprs", ".agpr_count:": "agprs", ".sgpr_count:": "sgprs",
            ".group_segment_fixed_size:": "lds_bytes", ".private_segment_fixed_size:": "scratch_bytes",
            ".vgpr_spill_count:": "vgpr_spills", ".sgpr_spill_count:": "sgpr_spills",
        }
        with open(asm) as f:
            for line in f:
                s = line.strip()
                if s.startswith("- "):  # the first key of a kernel's metadata entry
                    s = s[2:].lstrip()
                for k, name in keys.items():
                    if s.startswith(k):
                        out[name] = int(s.split()[-1])
        return out
