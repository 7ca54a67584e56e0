"""Builds libladder_hip.so (gfx950) from csrc/*.hip with plain hipcc: no torch headers, no cmake.

    python build.py            # compile what changed, link
    python build.py --force    # recompile everything

The shared library lands next to the Python package (gpt_fast/libladder_hip.so), in-tree, so that
it travels with the sources to a GPU machine.  hipcc cross-compiles without a GPU."""
import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "gpt_fast", "libladder_hip.so")
PROF_LIB = os.path.join(HERE, "gpt_fast", "libladder_hip_prof.so")
BAND_PROF_LIB = os.path.join(HERE, "gpt_fast", "libladder_hip_bandprof.so")
HEADERS = [os.path.join(CSRC, h) for h in ("lr_common.h", "attn_decode_item.h", "stream_band.h")] + \
    [os.path.join(HERE, "..", "include", "ladder_hip.h")]
# sources that compile another source under a switch
INCLUDES = {"ladder_step_fp8.hip": [os.path.join(CSRC, "ladder_step.hip")]}

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # packed-fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# per-source additions: the prefill attention rescales its matrix-core accumulators with vector instructions; kept
# in ordinary vector registers (not the accumulation registers) that costs no copies
PER_SOURCE_FLAGS = {"attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force, extra=(), suffix=""):
    obj = os.path.join(OBJ, os.path.basename(src).replace(".hip", suffix + ".o"))
    if not force and not _stale(obj, [src] + HEADERS + INCLUDES.get(os.path.basename(src), [])):
        return obj, False
    cmd = ["hipcc"] + FLAGS + PER_SOURCE_FLAGS.get(os.path.basename(src), []) + list(extra) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj, True


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        res = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in res]
    if force or any(c for _, c in res) or _stale(LIB, objs):
        cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB) / 1e6:.1f} MB) from {len(srcs)} sources")
    return LIB


def _build_variant(lib, sources, define, suffix, force, verbose):
    """`lib` = the product objects, with `sources` recompiled under `define`."""
    build(force=force, verbose=False)
    res = [_compile(os.path.join(CSRC, f), force, (define,), suffix) for f in sources]
    changed = any(c for _, c in res)
    objs = [os.path.join(OBJ, f.replace(".hip", ".o")) for f in sorted(os.listdir(CSRC))
            if f.endswith(".hip") and f not in sources] + [o for o, _ in res]
    if force or changed or _stale(lib, objs):
        r = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs,
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {lib}")
    return lib


def build_step_profile(force=False, verbose=True):
    """A second library, gpt_fast/libladder_hip_prof.so, whose decode-step kernels (bf16 and e4m3 weights) record
    wall-clock stamps per workgroup and phase (-DLR_STEP_PROFILE; read by step_phases.py).  The product library
    carries none of it."""
    return _build_variant(PROF_LIB, ("ladder_step.hip", "ladder_step_fp8.hip"), "-DLR_STEP_PROFILE", "_prof", force,
                          verbose)


def build_band_profile(force=False, verbose=True):
    """gpt_fast/libladder_hip_bandprof.so: the weight-streaming band kernel of lr_linear_multi records wall-clock
    stamps per wave (-DLR_BAND_PROFILE; read by band_phases.py).  The product library carries none of it."""
    return _build_variant(BAND_PROF_LIB, ("stream_gemm.hip",), "-DLR_BAND_PROFILE", "_bandprof", force, verbose)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--profile-step", action="store_true",
                    help="also build libladder_hip_prof.so (decode-step kernel with per-phase time stamps)")
    ap.add_argument("--profile-bands", action="store_true",
                    help="also build libladder_hip_bandprof.so (band kernel with per-wave time stamps)")
    args = ap.parse_args()
    build(force=args.force)
    if args.profile_step:
        build_step_profile(force=args.force)
    if args.profile_bands:
        build_band_profile(force=args.force)
