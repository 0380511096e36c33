"""Builds amct_amd/lib/libamct_hip.so from csrc/*.hip with hipcc for gfx950.

Run as `python -m amct_amd.build`.  hipcc cross-compiles without a GPU.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libamct_hip.so")
OBJDIR = os.path.join(LIBDIR, "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",                 # every fp32 op rounds separately, as the eager reference does
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


# Kernels whose s_waitcnt vmcnt values are counted by hand (inline-asm loads with a fixed number of operations per
# iteration): a register spill would add scratch loads and stores to that count and make them read registers before
# their data has landed.  The build refuses such a kernel instead of shipping it.
NO_SPILL = ("w8a8_tile_", "w4a16_tile_")
# Kernels that are built around "every load of a wave in flight at once" at a fixed register budget (16 waves per
# block: 128 registers).  A spill there costs speed, not correctness: reported, the build goes on.
REPORT_SPILL = ("_stream<", "w4a16_wave<")
_TAG = "[-Rpass-analysis=kernel-resource-usage]"


def _spilling_kernels(remarks, families=NO_SPILL):
    """Names of kernels of `families` for which the compiler reports spilled vector registers or scratch memory."""
    bad, name = [], None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif name and any(k in name for k in families):
            for key in ("VGPRs Spill:", "ScratchSize [bytes/lane]:"):
                if key in line and int(line.split(key)[1].split("[")[0].strip()) != 0:
                    bad.append("{} ({} {})".format(name, key, line.split(key)[1].split("[")[0].strip()))
    return sorted(set(bad))


def _without_resource_remarks(text):
    """Compiler output minus the resource-usage remarks and their source-context lines; warnings and errors keep
    theirs."""
    keep, skipping = [], False
    for line in text.splitlines():
        if _TAG in line:
            skipping = True
            continue
        if "warning:" in line or "error:" in line or "note:" in line:
            skipping = False
        elif skipping and (line.strip().startswith(("|", "^")) or " | " in line or "__launch_bounds__" in line or not line.strip()):
            continue
        else:
            skipping = False
        keep.append(line)
    return "\n".join(keep)


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.basename(src)[:-4] + ".o")
    check = os.path.basename(src).startswith("gemm_")
    cmd = [HIPCC] + FLAGS + (["-Rpass-analysis=kernel-resource-usage"] if check else []) + ["-c", src, "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    out = p.stdout + p.stderr
    if check and p.returncode == 0:
        bad = _spilling_kernels(out)
        if bad:
            return src, obj, 1, "kernels with hand-counted waits must not spill:\n  " + "\n  ".join(bad)
        slow = _spilling_kernels(out, REPORT_SPILL)
        out = _without_resource_remarks(out)
        if slow:
            out += "\nwarning: weight-streaming kernels that spill (slower, still correct):\n  " + "\n  ".join(slow)
    return src, obj, p.returncode, out


def build_library(verbose=True, jobs=8):
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, out in ex.map(_compile, srcs):
            msgs = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if rc != 0:
                raise RuntimeError("hipcc failed on {}:\n{}".format(src, out))
            if verbose:
                print("compiled", os.path.basename(src), flush=True)
                if msgs.strip() and "warning" in msgs:
                    print(msgs)
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stdout + p.stderr)
    if verbose:
        print("linked", LIB, flush=True)
    return LIB


if __name__ == "__main__":
    build_library()
    sys.exit(0)
