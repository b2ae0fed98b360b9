"""Builds libtorchode_amd.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m torchode_amd.build

hipcc cross-compiles without a GPU.  The library is written in-tree, next to
this file, so that it travels with the source tree.  Flags that matter for
results: floating point contraction is off (only the fma calls spelled out in the
sources fuse), float32 division and square root are the correctly rounded ones,
denormals are kept, and packed-FP32 instruction selection is disabled.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtorchode_amd.so")
OPS_LIB = os.path.join(HERE, "libtorchode_amd_ops.so")  # torch.ops.torchode_amd.*: PyTorch operators over the C ABI
OBJ = os.path.join(HERE, "build")

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-pass-failed",  # (a requested unrolling of a loop whose length only some instantiations know at compile time)
]  # fmt: skip

# (source, object name, extra defines)
UNITS = [
    ("tode_api.hip", "tode_api.o", []),
    ("tode_persistent.hip", "tode_persistent_f32.o", ["-DTODE_INSTANTIATE_F32=1"]),
    ("tode_persistent.hip", "tode_persistent_f64.o", ["-DTODE_INSTANTIATE_F64=1"]),
    ("tode_persistent.hip", "tode_persistent_t64_y32.o", ["-DTODE_INSTANTIATE_T64_Y32=1"]),
    ("tode_persistent.hip", "tode_persistent_t32_y64.o", ["-DTODE_INSTANTIATE_T32_Y64=1"]),
    ("tode_persistent.hip", "tode_persistent_f32_record.o", ["-DTODE_INSTANTIATE_F32=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_persistent.hip", "tode_persistent_f64_record.o", ["-DTODE_INSTANTIATE_F64=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_persistent.hip", "tode_persistent_t64_y32_record.o", ["-DTODE_INSTANTIATE_T64_Y32=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_persistent.hip", "tode_persistent_t32_y64_record.o", ["-DTODE_INSTANTIATE_T32_Y64=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_fast.hip", "tode_fast_f32.o", ["-DTODE_INSTANTIATE_F32=1"]),
    ("tode_fast.hip", "tode_fast_f64.o", ["-DTODE_INSTANTIATE_F64=1"]),
    ("tode_fast.hip", "tode_fast_f32_record.o", ["-DTODE_INSTANTIATE_F32=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_fast.hip", "tode_fast_f64_record.o", ["-DTODE_INSTANTIATE_F64=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_pair.hip", "tode_pair_f32.o", ["-DTODE_INSTANTIATE_F32=1"]),
    ("tode_pair.hip", "tode_pair_f64.o", ["-DTODE_INSTANTIATE_F64=1"]),
    ("tode_pair.hip", "tode_pair_f32_record.o", ["-DTODE_INSTANTIATE_F32=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_pair.hip", "tode_pair_f64_record.o", ["-DTODE_INSTANTIATE_F64=1", "-DTODE_INSTANTIATE_RECORD=1"]),
    ("tode_stepwise.hip", "tode_stepwise.o", []),
    ("tode_backward.hip", "tode_backward_f32.o", ["-DTODE_INSTANTIATE_F32=1"]),
    ("tode_backward.hip", "tode_backward_f64.o", ["-DTODE_INSTANTIATE_F64=1"]),
    ("tode_ops.hip", "tode_ops.o", []),
    ("tode_grid.hip", "tode_grid.o", []),
    ("tode_mlp.hip", "tode_mlp.o", []),
]


def source_hash() -> str:
    """sha256 over the library's sources (csrc/*, include/torchode_amd.h) and the compiler flags, in a fixed order.
    Compiled into the library (``tode_source_hash``) so that a loader can tell whether the file it found was built
    from the sources lying next to it."""
    import hashlib

    h = hashlib.sha256()
    files = sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith((".hip", ".h", ".cpp")))
    files.append(os.path.join(os.path.dirname(HERE), "include", "torchode_amd.h"))
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update(repr((FLAGS, UNITS)).encode())
    return h.hexdigest()


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"  # host pass does not know the AMDGPU feature
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{r.stdout}\n{err}")
    return err


def build_library(force: bool = True, verbose: bool = False) -> str:
    """Compiles every translation unit and links the shared library.  Returns its path."""
    if not force and os.path.exists(LIB):
        return LIB
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()

    digest = source_hash()

    def compile_unit(unit):
        src, obj, defs = unit
        out = os.path.join(OBJ, obj)
        if src == "tode_api.hip":
            defs = [*defs, f'-DTODE_SOURCE_HASH="{digest}"']
        msg = _run([hipcc, *FLAGS, *defs, "-c", os.path.join(CSRC, src), "-o", out])
        if verbose and msg.strip():
            print(msg, file=sys.stderr)
        return out

    with ThreadPoolExecutor(max_workers=min(8, len(UNITS) + 1)) as pool:
        ops_object = pool.submit(compile_ops_object)  # (host code only, done long before the kernels)
        checked = pool.submit(check_units_under_register_pressure)
        objs = list(pool.map(compile_unit, UNITS))
        ops_object = ops_object.result()
        checked.result()
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-Wno-unused-command-line-argument", "-o", LIB, *objs])
    link_ops_library(ops_object)
    return LIB


def compile_ops_object() -> str:
    """Compiles csrc/tode_torch_ops.cpp (host code only: PyTorch's headers, no kernel) to an object file."""
    import torch
    from torch.utils import cpp_extension

    out = os.path.join(OBJ, "tode_torch_ops.o")
    includes = [f"-I{p}" for p in cpp_extension.include_paths(device_type="cuda")] + ["-I/opt/rocm/include"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}", *includes,
          "-c", os.path.join(CSRC, "tode_torch_ops.cpp"), "-o", out])  # fmt: skip
    return out


def link_ops_library(obj=None) -> str:
    """Links the operator library against PyTorch's libraries and against libtorchode_amd.so, which it finds next to itself."""
    import torch

    if obj is None:
        obj = compile_ops_object()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    _run(["g++", "-shared", "-fPIC", obj, "-o", OPS_LIB, f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
          f"-L{HERE}", "-l:libtorchode_amd.so", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"])  # fmt: skip
    return OPS_LIB


def emit_assembly(directory: str, units=None) -> list:
    """The device code of every translation unit (or of ``units``, object names) as assembly text under ``directory``,
    compiled with the flags of the build.  Returns the paths."""
    os.makedirs(directory, exist_ok=True)
    hipcc = _hipcc()
    chosen = [u for u in UNITS if units is None or u[1] in units]

    def emit(unit):
        src, obj, defs = unit
        path = os.path.join(directory, obj[:-2] + ".s")
        _run([hipcc, *FLAGS, *defs, "-S", "--offload-device-only", os.path.join(CSRC, src), "-o", path])
        return path

    with ThreadPoolExecutor(max_workers=min(8, len(chosen) + 1)) as pool:
        return list(pool.map(emit, chosen))


# The units whose kernels keep whole per-sample arrays in registers (up to 256 of them, some in accumulation
# registers): where the compiler has been seen to place copies ahead of the execution mask's restore.
UNITS_UNDER_REGISTER_PRESSURE = ("tode_backward_f32.o", "tode_backward_f64.o")


def check_units_under_register_pressure() -> None:
    """Part of every build: the device assembly of those units is searched for the miscompilation described at
    ``copies_ahead_of_the_exec_restore``; a hit fails the build, since the library would load and run and return
    wrong gradients without any error."""
    for path in emit_assembly(os.path.join(OBJ, "asm"), UNITS_UNDER_REGISTER_PRESSURE):
        hits = copies_ahead_of_the_exec_restore(path)
        if hits:
            raise RuntimeError(f"{path}: register copies ahead of the restore of the execution mask (kernel, line, copies): {hits[:5]}")


def copies_ahead_of_the_exec_restore(assembly_path: str) -> list:
    """Looks through a unit's device assembly for a block that starts with copies of vector registers into
    accumulation registers (or spill stores) and only then restores the execution mask (``s_or_b64 exec, exec, ...``
    at the end of a divergent region).  Such copies run for the lanes that went through the region only, and a lane
    that skipped it continues with whatever the copy's target held before: wrong values without any error.  This
    compiler has placed copies like that in kernels under high register pressure.  Returns (kernel, line, count)."""
    import re

    lines = open(assembly_path).read().split("\n")
    found, kernel = [], None
    for n, line in enumerate(lines):
        name = re.match(r"^(_Z\w+):", line)
        if name:
            kernel = name.group(1)
        if not re.match(r"^\.LBB\d+_\d+:", line):
            continue
        copies = 0
        for text in lines[n + 1 : n + 64]:
            text = text.strip()
            if text.startswith((".LBB", "s_branch", "s_endpgm")) or "s_cbranch" in text:
                break
            if text.startswith("s_or_b64 exec, exec"):
                if copies:
                    found.append((kernel, n + 1, copies))
                break
            if text.startswith(("v_accvgpr_write", "scratch_store", "buffer_store")):
                copies += 1
    return found


if __name__ == "__main__":
    print(build_library(force=True, verbose=True))
