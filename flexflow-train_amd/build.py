"""Build recipe for libffk.so (the gfx950 operator-kernel library).

Every ``csrc/*.hip`` file is compiled to an object with hipcc for gfx950 and
the objects are linked into ``flexflow-train_amd/libffk.so`` next to this
file.  hipcc cross-compiles without a GPU, so this runs anywhere the ROCm
toolchain is installed.  Usage: ``python flexflow-train_amd/build.py [-j N]``.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libffk.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 instructions.
HIP_FLAGS = [
    "--offload-arch=" + ARCH,
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(HERE, "..", "include"),
]


# Per-file additions.  attention.hip: its backward kernels keep 128-160
# accumulator registers live across the loop; by default the compiler selects
# the MFMA form whose accumulators sit in accumulation registers and then
# copies every accumulator in and out of them around each step (several hundred
# moves per step).  Forcing the ordinary-register form removes the copies.
# optimizer.hip, loss.hip: these kernels promise the bits of the reference's CPU
# evaluation, where every fp32 operation is rounded on its own; the device
# compiler's default contracts a * b + c into one fused operation.
EXTRA_FLAGS = {
    "attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "attention_fwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form", "-fno-honor-nans"],
    "attention_bwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "optimizer.hip": ["-ffp-contract=off"],
    "loss.hip": ["-ffp-contract=off"],
}


def _sources():
    return sorted(
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip")
    )


def _headers_mtime():
    latest = 0.0
    for d in (CSRC, os.path.join(HERE, "..", "include")):
        for f in os.listdir(d):
            if f.endswith(".h"):
                latest = max(latest, os.path.getmtime(os.path.join(d, f)))
    return latest


def _compile_one(src, force):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    if (
        not force
        and os.path.exists(obj)
        and os.path.getmtime(obj) > max(os.path.getmtime(src), _headers_mtime())
    ):
        return obj, ""
    cmd = [HIPCC] + HIP_FLAGS + EXTRA_FLAGS.get(os.path.basename(src), []) + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(
        ln for ln in (proc.stdout + proc.stderr).splitlines()
        if "packed-fp32-ops" not in ln
    )
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build(jobs=8, force=True, verbose=False):
    """Compile every kernel source and link libffk.so. Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = _sources()
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for obj, log in pool.map(lambda s: _compile_one(s, force), srcs):
            objs.append(obj)
            if verbose and log.strip():
                print(log)
    cmd = [HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_PATH] + objs
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout + proc.stderr)
    return LIB_PATH


if __name__ == "__main__":
    jobs = 8
    force = True
    args = sys.argv[1:]
    if "-j" in args:
        jobs = int(args[args.index("-j") + 1])
    if "--incremental" in args:
        force = False
    print(build(jobs=jobs, force=force, verbose=True))
