"""Builds libcoeus_mi355x.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m coeus_amd.build [--force]

Every .hip file under coeus_amd/csrc is compiled to an object file (in parallel) and linked
into coeus_amd/libcoeus_mi355x.so.  hipcc cross-compiles for gfx950 without a GPU present.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libcoeus_mi355x.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 VALU instructions are disabled on purpose: some of their forms have produced wrong
# results on the target machines
# Kernel-argument preload: the first 16 dwords of a kernel's arguments arrive in scalar registers with
# the wave instead of through loads at its start, so the first weight requests of a decode kernel go
# out a little earlier (7B batch-1 decode matmuls 8.83 -> 8.75 us per launch, the step 0.5-1 % faster,
# same box, alternating).
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def _needs(src, obj, deps):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in [src] + deps)


# files whose arithmetic must match the CPU bit for bit: no FMA contraction
EXACT = {"weights.hip": ["-ffp-contract=off"], "sample.hip": ["-ffp-contract=off"]}


def _compile(src, obj):
    cmd = [HIPCC] + FLAGS + EXACT.get(os.path.basename(src), []) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32-ops feature: harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, r.returncode, err


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    deps = glob.glob(os.path.join(CSRC, "*.hpp")) + [os.path.join(HERE, "..", "include", "coeus.h")]
    jobs = []
    objs = []
    for s in srcs:
        o = os.path.join(OBJ, os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        if force or _needs(s, o, deps):
            jobs.append((s, o))
    failed = False
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        for src, rc, err in ex.map(lambda so: _compile(*so), jobs):
            if verbose:
                print(f"[hipcc] {os.path.basename(src)} rc={rc}")
            if err.strip() and (rc != 0 or verbose):
                print(err, file=sys.stderr)
            failed |= rc != 0
    if failed:
        raise RuntimeError("hipcc failed")
    if jobs or force or not os.path.exists(LIB):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        subprocess.check_call(cmd)
        if verbose:
            print(f"[link] {LIB}")
    return LIB


# The sources without device code (errors, configuration, parameter layout, .rustllm files, the
# tokenizer): what the sanitizer build of the host logic is made of.
HOST_ONLY = ["host.hip", "rustllm_file.hip", "bpe.hip"]
HOST_ASAN_LIB = os.path.join(OBJ, "libcoeus_host_asan.so")


def asan_runtime():
    """Path of the address sanitizer runtime of the compiler that hipcc drives."""
    r = subprocess.run([HIPCC, "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True, text=True)
    path = r.stdout.strip()
    return path if os.path.isabs(path) and os.path.exists(path) else None


def build_host_sanitized(verbose=False):
    """Builds the host-only sources with AddressSanitizer + UndefinedBehaviorSanitizer on the host
    pass (`-Xarch_host -fsanitize=...`; device code is never sanitized) into
    coeus_amd/build/libcoeus_host_asan.so.  A process that loads it needs the sanitizer runtime
    preloaded (asan_runtime())."""
    os.makedirs(OBJ, exist_ok=True)
    srcs = [os.path.join(CSRC, f) for f in HOST_ONLY]
    cmd = ([HIPCC] + FLAGS + ["-O1", "-g", "-fno-omit-frame-pointer", "-Xarch_host", "-fsanitize=address",
                              "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=undefined",
                              "-shared-libsan", "-shared", "-o", HOST_ASAN_LIB] + srcs)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print("\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l), file=sys.stderr)
    if r.returncode != 0:
        raise RuntimeError("sanitizer build failed")
    return HOST_ASAN_LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
