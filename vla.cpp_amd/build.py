"""Builds libvla.so (HIP kernels + C ABI + C++ host layer) for gfx950 with hipcc."""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libvla.so")
OBJ = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc"), "-I" + os.path.join(HERE, "host"),
    # never let the compiler form packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")) + glob.glob(os.path.join(HERE, "host", "*.cpp")))


# Kernels that keep registers "in flight" between an inline-assembly load and its wait must
# not spill: a spilled in-flight register is stored before its data arrives and reused while
# the load is still due.  Their scratch size is read from the compiler's resource remarks.
NO_SPILL_KERNELS = {"gemm.hip": ["ternary_gemm_x16_kernel"], "dit_self.hip": ["dit_self_block_kernel"]}


def _check_no_spill(src, remarks):
    for kernel in NO_SPILL_KERNELS.get(os.path.basename(src), []):
        lines = remarks.splitlines()
        seen = False
        for i, l in enumerate(lines):
            if "Function Name:" in l and kernel in l:
                for m in lines[i:i + 40]:
                    if "ScratchSize [bytes/lane]:" in m:
                        seen = True
                        size = int(m.split("ScratchSize [bytes/lane]:")[1].split()[0])
                        if size != 0:
                            raise RuntimeError("%s spills %d bytes per lane: its in-flight registers are not safe" % (kernel, size))
                        break
        if not seen:
            raise RuntimeError("no resource remarks for %s in %s" % (kernel, src))


# Per-file compiler options.  dit_self.hip: accumulators of its MFMAs stay in the ordinary
# vector registers; left to itself the compiler parks them in the accumulation registers and
# copies them back and forth around every MFMA (1300 copies in the K loop).
EXTRA_FLAGS = {"dit_self.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    extra = ["-Rpass-analysis=kernel-resource-usage"] if os.path.basename(src) in NO_SPILL_KERNELS else []
    extra = extra + EXTRA_FLAGS.get(os.path.basename(src), [])
    cmd = [HIPCC] + FLAGS + extra + ["-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if os.path.basename(src) in NO_SPILL_KERNELS:
        _check_no_spill(src, err)
        # the remarks are not diagnostics: drop them (and their source excerpts) from what verbose builds print
        keep, skip = [], 0
        for l in err.splitlines():
            if "-Rpass-analysis=kernel-resource-usage" in l:
                skip = 2
                continue
            if skip:
                skip -= 1
                continue
            keep.append(l)
        err = "\n".join(keep)
    return obj, err


def build(verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [o for o, _ in results]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
