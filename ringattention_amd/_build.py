"""Builds libringattn.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc, and the torch
front end libringattn_torch.so (host code only) with the host compiler."""
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
# RINGATTN_LIB: load another build of the library instead (the sanitized host build of the CPU tests)
LIB_PATH = os.environ.get("RINGATTN_LIB") or os.path.join(PKG_DIR, "libringattn.so")

TORCH_LIB_PATH = os.path.join(PKG_DIR, "libringattn_torch.so")

SOURCES = ["ringattn_kernels.hip", "ringattn_walk.hip", "ringattn_walk64.hip", "ringattn_api.hip", "ringattn_datagen.cpp"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-pthread", "-Wno-inline-asm",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


_TOOLCHAIN = None


def toolchain_id():
    """What else a build product depends on: the compile flags, the compiler and (for the torch front end) torch."""
    global _TOOLCHAIN
    if _TOOLCHAIN is None:
        hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
        try:
            ver = subprocess.run([hipcc, "--version"], capture_output=True, text=True).stdout
        except OSError:
            ver = "no hipcc"
        try:
            import torch
            tv = torch.__version__
        except Exception:
            tv = "no torch"
        _TOOLCHAIN = "\n".join(HIPCC_FLAGS) + "\n" + ver + "\n" + tv
    return _TOOLCHAIN


def source_id(paths):
    """sha256 over the given files, the compile flags and the toolchain versions: what a build product was made from."""
    import hashlib
    h = hashlib.sha256()
    for path in sorted(paths):
        with open(path, "rb") as f:
            h.update(os.path.basename(path).encode() + b"\0" + f.read())
    h.update(toolchain_id().encode())
    return h.hexdigest()


def library_sources():
    return [os.path.join(CSRC, s) for s in SOURCES] + [os.path.join(CSRC, "ringattn_kernels.h"), os.path.join(CSRC, "ringattn_device.h"),
                                                       os.path.join(CSRC, "ringattn_walk64_loop.inc"),
                                                       os.path.join(CSRC, "ringattn_walk64_loop_d64.inc"),
                                                       os.path.join(REPO_DIR, "include", "ringattn.h")]


def is_current(product, sources):
    """True if `product` exists and its stamp file names exactly these sources' contents."""
    stamp = product + ".stamp"
    if not (os.path.exists(product) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_id(sources)


def write_stamp(product, sources):
    with open(product + ".stamp", "w") as f:
        f.write(source_id(sources) + "\n")


def build_library(verbose=False):
    """Compile every HIP source of the package into libringattn.so.  Always recompiles."""
    if os.environ.get("RINGATTN_LIB"):
        raise RuntimeError("RINGATTN_LIB names a library built elsewhere: not overwriting it (unset it to build the package's own)")
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: cannot build libringattn.so")
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + ["-I", os.path.join(REPO_DIR, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stderr)
    os.replace(tmp, LIB_PATH)
    write_stamp(LIB_PATH, library_sources())
    return LIB_PATH


def torch_shim_sources():
    return [os.path.join(CSRC, "ringattn_torch.cpp"), os.path.join(REPO_DIR, "include", "ringattn.h")]


def harness_sources():
    return [os.path.join(CSRC, "reference_harness.cpp"), os.path.join(REPO_DIR, "include", "ringattn.h")]


def build_torch_shim(verbose=False):
    """Compile csrc/ringattn_torch.cpp (dispatcher op ringattn::fwd on top of the C ABI) against
    the installed torch.  Host code only; links libringattn.so by relative rpath.  Always recompiles."""
    import torch
    from torch.utils import cpp_extension
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("g++ not found: cannot build libringattn_torch.so")
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("build libringattn.so first")
    tmp = TORCH_LIB_PATH + ".tmp"
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}"]
    for inc in cpp_extension.include_paths("cuda") + [os.path.join(REPO_DIR, "include")]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "ringattn_torch.cpp"), "-o", tmp, "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu",
            "-ltorch_hip", "-ltorch", "-L", PKG_DIR, "-l:libringattn.so", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("torch shim build failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stderr)
    os.replace(tmp, TORCH_LIB_PATH)
    write_stamp(TORCH_LIB_PATH, torch_shim_sources())
    return TORCH_LIB_PATH


def sanitizer_runtime():
    """Path of the AddressSanitizer runtime of hipcc's clang (to be preloaded into a python that
    loads a sanitized library)."""
    clang = os.path.join(os.path.dirname(os.path.realpath(shutil.which("hipcc") or "/opt/rocm/bin/hipcc")), "..",
                         "lib", "llvm", "bin", "clang")
    if not os.path.exists(clang):
        clang = "/opt/rocm/lib/llvm/bin/clang"
    res = subprocess.run([clang, "--print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True)
    path = res.stdout.strip()
    if res.returncode != 0 or not os.path.isabs(path) or not os.path.exists(path):
        raise RuntimeError("AddressSanitizer runtime of hipcc's clang not found")
    return clang, path


def build_sanitized_library(out_dir):
    """The library with its HOST code (validation, schedule, plan lifetime, data generator, launch
    stubs) under AddressSanitizer and UndefinedBehaviorSanitizer, for the CPU tests.  The sanitizer
    flags are given to the host compilation only (-Xarch_host); the device code is the usual one."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = os.path.join(out_dir, "libringattn_san.so")
    cmd = [hipcc] + [f for f in HIPCC_FLAGS if f != "-O3"] + [
        "-O1", "-g", "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
        "-Xarch_host", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-shared-libsan",
        "-I", os.path.join(REPO_DIR, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    return out


HARNESS_PATH = os.path.join(PKG_DIR, "reference_harness")


def build_harness():
    """Compile csrc/reference_harness.cpp (the reference's main() on the C ABI; host code linked to libringattn.so)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, "-O2", "-std=c++17", "-I", os.path.join(REPO_DIR, "include"), os.path.join(CSRC, "reference_harness.cpp"),
           "-o", HARNESS_PATH, "-L", PKG_DIR, "-l:libringattn.so", "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    write_stamp(HARNESS_PATH, harness_sources())
    return HARNESS_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_harness())
    print(build_torch_shim(verbose=True))
