"""Build recipe for libgridnet_hip.so and the benchmark's libgridnet_probe.so (gfx950 only, hipcc,
in-tree).

Usage: ``python -m gridnet_amd.build`` or ``gridnet_amd.build.build()``.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libgridnet_hip.so")
SOURCES = ["api.hip", "step_generic.hip", "step_fast.hip", "fwd_rows.hip", "bwd_rows.hip", "cross_rows.hip", "chain_bwd.hip", "gated_generic.hip", "gated_fast.hip", "layernorm.hip"]
# machine ceilings for bench.py: not part of the product library (it allocates and synchronises)
PROBE_LIB = os.path.join(HERE, "libgridnet_probe.so")
PROBE_SOURCES = ["probe.hip"]

# -packed-fp32-ops is switched OFF on purpose: hipcc -O3 otherwise forms v_pk_*_f32 from
# ordinary float code.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# per source file, on top of FLAGS
FILE_FLAGS = {
    # chain_bwd.hip posts an arrival with an atomic add from one lane and reads the returned count
    # an iteration later; the atomic optimizer would make it a wave reduction that waits at once
    "chain_bwd.hip": ["-mllvm", "-amdgpu-atomic-optimizer-strategy=None"],
}


def build(verbose: bool = True, extra_flags=(), out=None, objdir=None) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = objdir or os.path.join(HERE, "build")
    out = out or LIB
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *FILE_FLAGS.get(src, []), *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(
            l for l in (res.stdout + res.stderr).splitlines()
            if "packed-fp32-ops" not in l  # the host pass does not know the device feature
        )
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + len(PROBE_SOURCES))) as pool:
        all_objs = list(pool.map(compile_one, SOURCES + PROBE_SOURCES))
    objs, probe_objs = all_objs[:len(SOURCES)], all_objs[len(SOURCES):]
    probe_out = os.path.join(os.path.dirname(out), os.path.basename(PROBE_LIB))
    for target, members in ((out, objs), (probe_out, probe_objs)):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *members, "-o", target]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
