"""Compile the HIP sources in csrc/ for gfx950 into

  khaosz_amd/lib/libastrai_q.so      the product: the C ABI declared in include/astrai_q.h, nothing else;
  khaosz_amd/lib/libastrai_q_lab.so  the same objects plus the measurement probes and the tile-forcing hook
                                     of csrc/aq_lab.h (the GEMM and GEMV sources rebuilt with -DAQ_LAB), for the
                                     benchmark's ceilings and for tests that pin a tile shape.

hipcc cross-compiles without a GPU.  Both depend on the HIP runtime only (no torch, no Python).

    python -m khaosz_amd.build [--if-stale] [--stall-counters]

--stall-counters builds the lab library's GEMM object with -DAQ_LAB_STALL as well: cycle counters inside the K
loop (waits at the stage barriers, loop, prologue, epilogue; read with aq_lab_read_clock).  They cost a few clock
reads per K step, so the default lab build leaves them out; the product library never has them.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "lib", "obj")
LIB = os.path.join(HERE, "lib", "libastrai_q.so")
LAB_LIB = os.path.join(HERE, "lib", "libastrai_q_lab.so")
SOURCES = ["abi.hip", "quant.hip", "gemm_mfma.hip", "gemv.hip", "attn_decode.hip", "attn_prefill.hip"]
# (source, object, extra flags) of the lab library's own objects; the other product objects are shared
LAB_SOURCES = [("gemm_mfma.hip", "gemm_mfma_lab.o", ["-DAQ_LAB"]), ("gemv.hip", "gemv_lab.o", ["-DAQ_LAB"]),
               ("lab.hip", "lab.o", [])]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # every fp32 operation rounds on its own (bit-exact parity with the CPU oracle)
    "-ffp-contract=off",
    # packed-fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _stale(out, deps):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = True, verbose: bool = False, stall_counters: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    lab_sources = [(src, obj, extra + (["-DAQ_LAB_STALL"] if stall_counters and src == "gemm_mfma.hip" else []))
                   for src, obj, extra in LAB_SOURCES]
    headers = [os.path.join(CSRC, "aq_common.h"), os.path.join(CSRC, "aq_rows.h"), os.path.join(CSRC, "aq_lab.h"),
               os.path.join(HERE, "..", "include", "astrai_q.h")]

    def compile_one(job):
        src, obj, extra = job if isinstance(job, tuple) else (job, job.replace(".hip", ".o"), [])
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ_DIR, obj)
        if force or _stale(o, [s] + headers):
            cmd = [HIPCC, *FLAGS, *extra, "-c", s, "-o", o]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr}")
            if verbose and r.stderr:
                # the host pass warns that it does not know the packed-fp32 feature: harmless
                print("\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l), file=sys.stderr)
        return o

    with ThreadPoolExecutor(max_workers=4) as ex:
        all_objs = list(ex.map(compile_one, SOURCES + lab_sources))
    objs, lab_only = all_objs[:len(SOURCES)], all_objs[len(SOURCES):]
    lab_objs = [o for o in objs if not o.endswith(("gemm_mfma.o", "gemv.o"))] + lab_only
    for lib, members in ((LIB, objs), (LAB_LIB, lab_objs)):
        if force or _stale(lib, members):
            cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *members]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    stall = "--stall-counters" in sys.argv
    print(build(force=stall or "--if-stale" not in sys.argv, verbose=True, stall_counters=stall))
