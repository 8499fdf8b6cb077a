"""Build libexodus_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage:  python build_hip.py
The library lands next to the Python loader (sinabs/exodus/libexodus_hip.so).  A second, small
library with the streaming probes that only bench.py uses (libexodus_bench_probes.so, next to this
script) is built in the same go; it is not part of the product.
"""
import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
SRCS = [os.path.join(HERE, "csrc", f) for f in ("exodus_hip.hip", "exodus_layer.hip", "exodus_hbm.hip")]
SRC = SRCS[0]
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT = os.path.join(HERE, "sinabs", "exodus", "libexodus_hip.so")
PROBE_SRC = os.path.join(HERE, "csrc", "bench_probes.hip")
PROBE_OUT = os.path.join(HERE, "libexodus_bench_probes.so")

# -ffp-contract=off : the forward recurrences must round every multiply and add separately
# -packed-fp32-ops disabled : keep the compiler from forming packed fp32 instructions
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wno-unused-command-line-argument",
]


def build(force: bool = True) -> str:
    deps = SRCS + [PROBE_SRC, os.path.join(HERE, "csrc", "exodus_common.hpp"), os.path.join(INCLUDE, "exodus_hip.h")]
    if (not force and os.path.exists(OUT) and os.path.exists(PROBE_OUT)
            and min(os.path.getmtime(OUT), os.path.getmtime(PROBE_OUT)) >= max(os.path.getmtime(d) for d in deps)):
        return OUT
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    # hipcc's host pass does not know the gfx-only target feature and says so; that line is harmless
    noise = "packed-fp32-ops"
    quiet = lambda text: "\n".join(l for l in text.splitlines() if noise not in l)
    compile_flags = [f for f in FLAGS if f != "-shared"]
    with tempfile.TemporaryDirectory() as tmp:
        # one hipcc process per translation unit, side by side, then one link
        objs = [os.path.join(tmp, os.path.basename(src) + ".o") for src in SRCS]
        procs = [subprocess.Popen([hipcc] + compile_flags + ["-I", INCLUDE, "-c", src, "-o", obj],
                                  stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
                 for src, obj in zip(SRCS, objs)]
        # the bench-only probes: one small translation unit, compiled and linked in one step
        procs.append(subprocess.Popen([hipcc] + FLAGS + ["-I", INCLUDE, PROBE_SRC, "-o", PROBE_OUT + ".tmp"],
                                      stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
        outputs = [proc.communicate()[0] for proc in procs]
        log = "\n".join(filter(None, (quiet(o).strip() for o in outputs)))
        if any(proc.returncode != 0 for proc in procs):
            sys.stderr.write(log + "\n")
            raise RuntimeError("hipcc failed compiling libexodus_hip.so / libexodus_bench_probes.so")
        link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT + ".tmp"] + objs,
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        log = "\n".join(filter(None, (log, quiet(link.stdout).strip())))
        if link.returncode != 0:
            sys.stderr.write(log + "\n")
            raise RuntimeError("hipcc failed linking libexodus_hip.so")
    if log.strip():
        sys.stderr.write(log + "\n")
    os.replace(OUT + ".tmp", OUT)
    os.replace(PROBE_OUT + ".tmp", PROBE_OUT)
    return OUT


if __name__ == "__main__":
    print(build(force=True))
