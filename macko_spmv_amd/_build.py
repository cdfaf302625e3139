"""Build recipes for the two native libraries of this package.

  libmacko_hip.so    torch-free HIP kernels behind the C ABI of include/macko_hip.h (gfx950)
  libmacko_torch.so  PyTorch-ROCm operator library that forwards to the C ABI
  libmacko_bench.so  the benchmark's own kernels (streaming-read yardstick, counter calibration)

Both are built in-tree (next to this file) unless MACKO_SPMV_BUILD_DIRECTORY names another
directory -- the same variable the upstream package reads for its JIT cache
(src/macko_spmv/__init__.py:12).  hipcc cross-compiles for gfx950 without a GPU present.

Run `python -m macko_spmv_amd._build` to (re)build them (`--devtools`: the tracing build and phase_trace).
"""
import os
import re
import shutil
import subprocess
import sys
import tempfile

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
_CSRC = os.path.join(_PKG, "csrc")
_INCLUDE = os.path.join(_ROOT, "include")

HIP_LIB = "libmacko_hip.so"
TORCH_LIB = "libmacko_torch.so"
BENCH_LIB = "libmacko_bench.so"  # kernels of bench.py only; the package never loads it
ARCH = "gfx950"

HIP_SOURCES = ["macko_spmv.hip", "macko_spmv_split.hip", "macko_compress.hip", "macko_runtime.hip", "macko_decode.hip"]
TORCH_SOURCES = ["macko_torch.cpp"]
BENCH_SOURCES = ["macko_bench_kernels.hip"]


def build_directory():
    d = os.environ.get("MACKO_SPMV_BUILD_DIRECTORY", "")
    if d:
        os.makedirs(d, exist_ok=True)
        return d
    return _PKG


def lib_paths():
    d = build_directory()
    return os.path.join(d, HIP_LIB), os.path.join(d, TORCH_LIB)


def _hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: a ROCm toolchain is required to build macko_spmv_amd")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed:\n" + " ".join(cmd) + "\n" + proc.stdout)
    if verbose and proc.stdout.strip():
        print(proc.stdout, flush=True)


_DEVICE_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17",
    # keep the compiler from forming packed fp32 VALU ops (device pass; the host pass ignores it)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    f"-I{_INCLUDE}", f"-I{_CSRC}",
]

# The SpMV kernels keep their in-flight loads in fixed VGPRs from a certain register up
# (kCompilerVgprs in their source files); compiler-generated code must stay below it.
# source file -> (kernel name, first fixed VGPR, first register of every ring slot)
TRACKED_KERNELS = {
    "macko_spmv.hip": ("spmv_stream_kernel", 78, (88, 92, 96, 100)),
    "macko_spmv_split.hip": ("spmv_split_kernel", 84, (94, 98)),
}


def check_stream_kernel_assembly(text, kernel_name="spmv_stream_kernel", fixed_base=78, slot_registers=(88, 92, 96, 100)):
    """`text`: lines of the assembly of one of the SpMV source files.  Checks two things the
    hand-tracked loads of every instantiation of `kernel_name` rely on: outside the hand-written asm
    blocks no instruction touches a VGPR >= fixed_base, and the compiler has put no vmcnt wait of its
    own right in front of a ring take (it does when one of its own loads may still be outstanding at
    the loop's back edge; such a wait also waits for the ring loads in flight and serialises the
    stream).  Also checks that no kernel of the file calls a function or uses scratch memory.
    Returns the number of kernels checked; raises RuntimeError on a violation."""
    kernel = None
    in_asm = False
    checked = 0
    recent_wait = None  # (line number, text) of the last compiler-generated vmcnt wait
    take = re.compile(r"v_mov_b32 \S+ v(%s)\b" % "|".join(str(r) for r in slot_registers))
    for number, line in enumerate(text):
        m = re.match(r"^(_Z\S*%s\S*):" % kernel_name, line)
        if m:
            kernel, in_asm, recent_wait = m.group(1), False, None
            checked += 1
            continue
        if kernel is None:
            continue
        if line.startswith(".Lfunc_end") or ".amdhsa_kernel" in line:
            kernel = None
        elif "#ASMSTART" in line:
            in_asm = True
        elif "#ASMEND" in line:
            in_asm = False
        elif in_asm:
            # a ring take copies out of its slot's registers after its own wait
            if recent_wait and number - recent_wait[0] <= 16 and take.search(line):
                raise RuntimeError(f"compiler-generated '{recent_wait[1]}' in front of a ring take in {kernel} "
                                   f"(assembly line {recent_wait[0] + 1})")
        else:
            code = line.split(";")[0]
            if re.match(r"^\s*\.L?BB\d+_\d+:", code):
                recent_wait = None  # a label: what follows is another block
            if re.search(r"s_waitcnt\b.*vmcnt\(", code):
                recent_wait = (number, code.strip())
            regs = [int(b) for _, b in re.findall(r"\bv\[(\d+):(\d+)\]", code)]
            regs += [int(a) for a in re.findall(r"\bv(\d+)\b", code)]
            if regs and max(regs) >= fixed_base:
                raise RuntimeError(f"compiler-generated code touches a fixed VGPR in {kernel}: {line.strip()}")
    if checked == 0:
        raise RuntimeError(f"no {kernel_name} found in the assembly; the register check is stale")
    # No kernel of these files may call a function or keep anything in scratch memory: a lambda of
    # the kernel that is not inlined takes its captures, the kernel's whole state, through memory
    # (measured: four times slower), and its code would not be covered by the checks above.
    for number, line in enumerate(text):
        code = line.split(";")[0]
        if re.search(r"\bs_swappc_b64\b|\bscratch_(load|store)_", code):
            raise RuntimeError(f"function call or scratch access in the assembly (line {number + 1}): {code.strip()}")
        m = re.search(r"\.amdhsa_private_segment_fixed_size\s+(\d+)", code)
        if m and int(m.group(1)) != 0:
            raise RuntimeError(f"a kernel uses {m.group(1)} bytes of scratch memory (assembly line {number + 1})")
    return checked


def verify_fixed_registers(verbose=False, extra_flags=()):
    """Compile the SpMV sources to assembly (with `extra_flags`, so that a build with other
    preprocessor settings is checked as it is built) and run check_stream_kernel_assembly on each."""
    checked = 0
    with tempfile.TemporaryDirectory() as tmp:
        for source, (kernel_name, fixed_base, slot_registers) in TRACKED_KERNELS.items():
            asm = os.path.join(tmp, source + ".s")
            _run([_hipcc(), *_DEVICE_FLAGS, *extra_flags, "--cuda-device-only", "-S", os.path.join(_CSRC, source),
                  "-o", asm], verbose)
            with open(asm) as f:
                checked += check_stream_kernel_assembly(f.read().splitlines(), kernel_name, fixed_base, slot_registers)
    return checked


def build_hip(verbose=False):
    """Builds libmacko_hip.so.  The library only reaches its final path once the generated code
    has passed the fixed-register check: an unchecked library must never be the one that loads."""
    out, _ = lib_paths()
    verify_fixed_registers(verbose)
    staging = out + ".building"
    cmd = [
        # only what include/*.h declare is exported
        _hipcc(), *_DEVICE_FLAGS, "-fvisibility=hidden", "-fPIC", "-shared",
        *[os.path.join(_CSRC, s) for s in HIP_SOURCES],
        "-o", staging,
    ]
    try:
        _run(cmd, verbose)
        os.replace(staging, out)
    finally:
        if os.path.exists(staging):
            os.remove(staging)
    return out


STAMP = "macko_build.stamp"


def source_digest():
    """Hash of everything the two libraries are built from (csrc/, include/, this recipe)."""
    import hashlib

    h = hashlib.sha256()
    files = [os.path.abspath(__file__)]
    for directory in (_CSRC, _INCLUDE):
        files += [os.path.join(directory, name) for name in sorted(os.listdir(directory))]
    for full in files:
        if os.path.isfile(full):
            h.update(os.path.basename(full).encode())
            with open(full, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def stamp_path():
    return os.path.join(build_directory(), STAMP)


def is_current():
    """True when both libraries exist and were built from the sources as they are now."""
    hip_lib, torch_lib = lib_paths()
    if not all(os.path.exists(f) for f in (hip_lib, torch_lib, bench_lib_path(), stamp_path())):
        return False
    with open(stamp_path()) as f:
        return f.read().strip() == source_digest()


def build_torch(verbose=False):
    import torch
    from torch.utils import cpp_extension as ce

    hip_lib, out = lib_paths()
    if not os.path.exists(hip_lib):
        build_hip(verbose)
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        _hipcc(), "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        "-Wno-unused-command-line-argument",
        f"-I{_INCLUDE}",
        *[f"-I{p}" for p in ce.include_paths("cuda")],
        *[os.path.join(_CSRC, s) for s in TORCH_SOURCES],
        "-x", "none",
        *[f"-L{p}" for p in ce.library_paths("cuda") if os.path.isdir(p)],
        f"-L{os.path.dirname(hip_lib)}",
        "-lmacko_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN",
        "-o", out,
    ]
    _run(cmd, verbose)
    return out


def bench_lib_path():
    return os.path.join(build_directory(), BENCH_LIB)


def build_bench(verbose=False):
    out = bench_lib_path()
    _run([_hipcc(), *_DEVICE_FLAGS, "-fPIC", "-shared", *[os.path.join(_CSRC, s) for s in BENCH_SOURCES], "-o", out],
         verbose)
    return out


def build_devtools(verbose=False):
    """Development tools, not part of the product and never loaded by it: a tracing build of the
    HIP library (phase stamps and launch-shape overrides, -DMACKO_DEV_HOOKS) and phase_trace,
    the program that prints per-wave phase tables from it.  Both land in macko_spmv_amd/devtools/."""
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "devtools")
    lib = os.path.join(here, "libmacko_hip_trace.so")
    tool = os.path.join(here, "phase_trace")
    verify_fixed_registers(verbose, extra_flags=("-DMACKO_DEV_HOOKS",))  # the stamps are code between the takes
    _run([_hipcc(), *_DEVICE_FLAGS, "-DMACKO_DEV_HOOKS", "-fPIC", "-shared",
          *[os.path.join(_CSRC, s) for s in HIP_SOURCES], "-o", lib], verbose)
    _run([_hipcc(), "--offload-arch=gfx950", "-O2", "-std=c++17", os.path.join(here, "phase_trace.hip"),
          "-ldl", "-o", tool], verbose)
    return lib, tool


def build_all(verbose=False):
    if os.path.exists(stamp_path()):
        os.remove(stamp_path())
    built = build_hip(verbose), build_torch(verbose)
    build_bench(verbose)
    with open(stamp_path(), "w") as f:
        f.write(source_digest() + "\n")
    return built


if __name__ == "__main__":
    build = build_devtools if "--devtools" in sys.argv else build_all
    for path in build(verbose="-q" not in sys.argv):
        print("built", path)
