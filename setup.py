"""Build of the MI355X (gfx950) kernels and their PyTorch-ROCm binding.

``python setup.py build_ext --inplace`` produces, inside ``areno_amd/accel/``:

* ``libareno_hip.so``  -- the HIP kernels behind a C ABI (``include/areno_hip.h``); every
  ``areno_amd/csrc/*.hip`` file is compiled by ``hipcc --offload-arch=gfx950`` directly (no hipify pass,
  no CUDA-compat headers) and linked into one shared library with no torch dependency;
* ``_areno_accel<ext-suffix>.so`` -- the thin pybind11 / ATen binding (``areno_amd/csrc/extension.cpp``),
  linked against ``libareno_hip.so`` through an ``$ORIGIN`` rpath.

Environment switches follow the reference's ``setup.py`` (l.15-24 there): ``ARENO_BUILD_EXT=0`` and
metadata-only commands skip the native build.  ``ARENO_HIPCC`` overrides the compiler,
``ARENO_BUILD_JOBS`` the number of parallel compile jobs.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

from setuptools import Extension, find_packages, setup
from setuptools.command.build_ext import build_ext

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "areno_amd" / "csrc"
OUT_DIR = ROOT / "areno_amd" / "accel"
GPU_ARCH = "gfx950"
_METADATA_COMMANDS = {"egg_info", "dist_info", "sdist"}

# Packed-FP32 VALU forms are disabled for all device code (they have given wrong results on the target pool).
HIP_DEVICE_FLAGS = [
    f"--offload-arch={GPU_ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-honor-nans",  # fmaxf as a bare v_max_f32 / v_max3_f32 (no canonicalising self-max); nothing here relies on NaN
    # leading scalar kernel arguments (up to 16 words) arrive in registers at wave start instead of through a fetch of
    # the argument block: the decode kernels put what their first loads are addressed with there
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    # matrix products accumulate in vector registers: left to itself the compiler puts the decode kernels'
    # accumulators into accumulation registers and copies all 36 of them out and back around the rescaling of every
    # tile step (117 copies per step at head dim 128); no kernel here needs more than the 256 vector registers
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-DARENO_DEVICE_FLAGS_OK=1",  # device_common.hpp refuses to compile without the two flags above
] + [f"-D{name}={os.environ[name]}" for name in ("ARENO_MFMA_NW", "ARENO_TRACE", "ARENO_MFMA_QUANT_OCC", "ARENO_MFMA_WIDE_OCC", "ARENO_PREFILL_WAVES") if os.environ.get(name)]  # fmt: skip


def _hipcc() -> str:
    cand = os.environ.get("ARENO_HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(cand):
        raise RuntimeError(
            "areno_amd build failed: hipcc was not found.\n"
            "Why: the gfx950 kernels are compiled by ROCm's hipcc.\n"
            "Next steps: install ROCm >= 7 and put /opt/rocm/bin on PATH, or set ARENO_HIPCC, or set "
            "ARENO_BUILD_EXT=0 for a metadata-only install."
        )
    return cand


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_kernels_library(build_temp: Path, jobs: int) -> Path:
    hipcc = _hipcc()
    build_temp.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    objects = [build_temp / (src.stem + ".o") for src in sources]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc, *HIP_DEVICE_FLAGS, "-I", str(ROOT / "include"), "-c", str(src), "-o", str(obj)])
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    lib = OUT_DIR / "libareno_hip.so"
    _run([hipcc, f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(lib), *map(str, objects)])
    return lib


def build_torch_binding(build_temp: Path) -> Path:
    import torch
    from torch.utils import cpp_extension

    hipcc = _hipcc()
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    target = OUT_DIR / f"_areno_accel{suffix}"
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    includes = [*cpp_extension.include_paths("cuda"), sysconfig.get_paths()["include"], str(ROOT / "include")]
    cmd = [hipcc, "-x", "c++", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_areno_accel",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]  # fmt: skip
    for inc in includes:
        cmd += ["-isystem" if "torch" in inc or "python" in inc else "-I", inc]
    cmd += [str(CSRC / "extension.cpp"), "-o", str(target), f"-L{OUT_DIR}", "-lareno_hip", f"-L{torch_lib}",
            "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]  # fmt: skip
    _run(cmd)
    return target


class BuildHip(build_ext):
    """Replaces the stock compiler driver: the sources are HIP, compiled by hipcc directly."""

    def run(self) -> None:
        jobs = int(os.environ.get("ARENO_BUILD_JOBS", str(min(8, os.cpu_count() or 1))))
        build_temp = Path(self.build_temp) / "areno_hip"
        lib = build_kernels_library(build_temp, jobs)
        ext = build_torch_binding(build_temp)
        print(f"built {lib}\nbuilt {ext}")
        if not self.inplace:
            dest = Path(self.build_lib) / "areno_amd" / "accel"
            dest.mkdir(parents=True, exist_ok=True)
            for f in (lib, ext):
                shutil.copy2(f, dest / f.name)


def _extensions():
    if any(arg in _METADATA_COMMANDS for arg in sys.argv[1:]):
        return [], {}
    if os.environ.get("ARENO_BUILD_EXT", "1").lower() in {"0", "false", "no", "off"}:
        return [], {}
    return [Extension("areno_amd.accel._areno_accel", sources=[])], {"build_ext": BuildHip}


ext_modules, cmdclass = _extensions()

setup(
    name="areno_amd",
    version="0.1.0",
    description="MI355X-native paged / quantized KV-cache attention ops with AReno's op signatures",
    packages=find_packages(include=["areno_amd", "areno_amd.*"]),
    package_data={"areno_amd.accel": ["*.so"]},
    ext_modules=ext_modules,
    cmdclass=cmdclass,
)
