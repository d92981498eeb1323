"""Builds libtpumlir_amd.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc."""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtpumlir_amd.so")
SOURCES = ["a16_kernels.hip", "a16_decode.hip", "a16_gemm.hip", "a16_kn.hip", "a16_plain.hip", "a16_wide.hip", "a16_rows32.hip", "top_a16.hip", "i8_kernels.hip", "cast_kernels.hip", "quant_kernels.hip", "dq_kernels.hip", "f8_kernels.hip", "workspace.hip", "capi.hip", "module.hip", "bench_kernels.hip"]
# packed fp32 VALU ops are switched off for every device translation unit
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# the decode kernel's leading 14 argument dwords are preloaded into SGPRs at wave launch (see a16_decode.hip)
# (the read-only kernel the benchmark takes its launch ceilings from gets the same treatment: a ceiling must not be
# handicapped against the kernel it bounds)
EXTRA_FLAGS = {"a16_decode.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"],
               "bench_kernels.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=6"]}

# Kernels that keep load requests in flight across their loop (issued by inline asm, waited for by hand-counted
# s_waitcnt) must not spill: the compiler takes a requested register for loaded, may store it to scratch and hand the
# register on, and the data then lands on the register's next user; and a spill's own memory instruction moves the
# count the waits rely on.  These files are compiled with the resource report on, and a spilling instance of such a
# kernel fails the build.
NO_SPILL = {"a16_rows32.hip": ("rows32", "rows16"), "a16_wide.hip": ("wide",), "i8_kernels.hip": ("rows32",),
            "f8_kernels.hip": ("rows32",)}
REPORT_FLAG = "-Rpass-analysis=kernel-resource-usage"


def _spilling_kernels(report, name_parts):
    """Names of the kernels in a resource report whose name holds one of name_parts and that use scratch memory."""
    bad = []
    for block in re.split(r"remark:\s+Function Name: ", report)[1:]:
        name = block.split()[0]
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", block)
        if any(part in name for part in name_parts) and m and int(m.group(1)) > 0:
            bad.append("%s (%s bytes/lane)" % (name, m.group(1)))
    return bad


def build_library(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = ["hipcc", *FLAGS, *EXTRA_FLAGS.get(src, []), *([REPORT_FLAG] if src in NO_SPILL else []), "-c",
               os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass does not know the AMDGPU feature flag and says so; drop that line
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if src in NO_SPILL:
            bad = _spilling_kernels(out, NO_SPILL[src])
            if bad:
                raise RuntimeError("%s: kernels with requests in flight must not spill:\n  %s" % (src, "\n  ".join(bad)))
            out = "\n".join(l for l in out.splitlines() if REPORT_FLAG not in l)
        if verbose and out.strip():
            print(out)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
