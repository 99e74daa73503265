"""Builds the CPU oracle (test infrastructure, never part of the product path).

  oracle/liboracle.so       <- oracle/attention_oracle.c   (gcc -O3 -fopenmp)

The reference's own path cannot be compiled here: csrc/ring_attention.cu needs nvcc,
CUTLASS/CuTe (an empty, un-fetched submodule) and NVSHMEM, and the file is truncated
(csrc/ring_attention.cu:244-248), so there is no oracle/_ref build.
"""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
# ORACLE_LIB: load another build instead (the sanitized one of tests/test_sanitizers.py)
LIB_PATH = os.environ.get("ORACLE_LIB") or os.path.join(HERE, "liboracle.so")


def build_oracle():
    gcc = shutil.which("gcc")
    if not gcc:
        raise RuntimeError("gcc not found: cannot build the oracle")
    tmp = LIB_PATH + ".tmp"
    cmd = [gcc, "-O3", "-march=x86-64-v3", "-fopenmp", "-fPIC", "-shared", "-std=c11",
           os.path.join(HERE, "attention_oracle.c"), "-o", tmp, "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    os.replace(tmp, LIB_PATH)
    with open(LIB_PATH + ".stamp", "w") as f:
        f.write(source_id() + "\n")
    return LIB_PATH


def source_id():
    import hashlib
    with open(os.path.join(HERE, "attention_oracle.c"), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def is_current():
    stamp = LIB_PATH + ".stamp"
    if not (os.path.exists(LIB_PATH) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_id()


def build_oracle_sanitized(clang, out_dir):
    """The oracle with AddressSanitizer + UndefinedBehaviorSanitizer, built with the clang whose
    sanitizer runtime the sanitized library uses as well (one runtime per process); no OpenMP."""
    out = os.path.join(out_dir, "liboracle_san.so")
    cmd = [clang, "-O1", "-g", "-fPIC", "-shared", "-std=c11", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-shared-libsan",
           os.path.join(HERE, "attention_oracle.c"), "-o", out, "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("clang failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    return out


if __name__ == "__main__":
    print(build_oracle())
