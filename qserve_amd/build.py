"""Build libqserve_amd.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m qserve_amd.build [--force]

hipcc cross-compiles without a GPU, so this runs in the authoring container as well as on the MI355X box.
The .so lands in qserve_amd/ (git-ignored, but shipped to the GPU box by gpurun).
"""
import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "libqserve_amd.so")
SOURCES = ["lib.hip", "gemm_w4a8.hip", "gemm_w4a8_lds.hip", "gemm_w4a8_tiled.hip", "gemm_w4a8_wide.hip", "gemm_w4a8_ring.hip", "gemm_w8a8.hip", "attention.hip", "attention_mfma.hip", "attention_mfma8.hip", "flash_prefill.hip", "fused_small.hip", "direct_allreduce.hip"]
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
         "-Wno-unused-variable", "-Wno-unused-but-set-variable"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (need ROCm >= 7.0 with the gfx950 target)")
    return exe


def _deps_mtime():
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs.append(os.path.join(os.path.dirname(HERE), "include", "qserve_amd.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def _compile(src, force, extra, build_dir):
    obj = os.path.join(build_dir, src.replace(".hip", ".o"))
    srcp = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(srcp), _deps_mtime())):
        return obj, False
    cmd = [hipcc(), *FLAGS, *extra, "-c", srcp, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
    return obj, True


def build(force=False, verbose=True, extra=(), timing=False):
    """timing=True: the measurement build (-DQS_TIMING: ablation switches that turn kernel parts off, timeline traces) ->
    libqserve_amd_timing.so from its own object directory; never loaded by the product (qserve_amd/_lib.py loads it only when
    QS_AMD_LIBRARY names it - scripts/)."""
    build_dir, lib = BUILD, LIB      # (locals: a timing build must not redirect later product builds of this process)
    if timing:
        build_dir, lib = os.path.join(HERE, "_build_timing"), os.path.join(HERE, "libqserve_amd_timing.so")
        extra = list(extra) + ["-DQS_TIMING"]
    os.makedirs(build_dir, exist_ok=True)
    extra = list(extra) + os.environ.get("QS_EXTRA_HIPCC_FLAGS", "").split()   # e.g. -DQS_RING_TRACE (timing tools)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        res = list(ex.map(lambda s: _compile(s, force, list(extra), build_dir), SOURCES))
    objs = [o for o, _ in res]
    rebuilt = any(r for _, r in res)
    if rebuilt or not os.path.exists(lib) or force:
        # (--no-undefined: a symbol one translation unit expects from another and does not get must fail HERE, not at dlopen)
        cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,--no-undefined", *objs, "-o", lib]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
        if verbose:
            print(f"[qserve_amd.build] linked {lib}")
    elif verbose:
        print(f"[qserve_amd.build] up to date: {lib}")
    return lib


# ---- libqserve_serve.so: the kernels of the paged serving engine (qserve_amd/serving) -------------------------------------------
# A library of its own: a model served by that engine needs these few translation units only, so its first start in a fresh
# checkout compiles them (a minute) and not the W4A8 GEMM / KV4 attention families above.
SERVE_CSRC = os.path.join(CSRC, "serve")
SERVE_BUILD = os.path.join(HERE, "_build_serve")
SERVE_LIB = os.path.join(HERE, "libqserve_serve.so")
SERVE_SOURCES = ["serve_rows.hip", "serve_attention.hip", "serve_attention_mfma.hip", "serve_moe.hip", "serve_moe_gemm.hip",
                 "serve_streams.hip", "serve_recurrent.hip"]
# packed-FP32 instructions off: the kernels' float statistics must not depend on how the compiler pairs them
SERVE_FLAGS = FLAGS + ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def serve_stale():
    """True if libqserve_serve.so is missing or older than one of its sources."""
    if not os.path.exists(SERVE_LIB):
        return True
    deps = [os.path.join(SERVE_CSRC, f) for f in os.listdir(SERVE_CSRC)]
    deps.append(os.path.join(os.path.dirname(HERE), "include", "qserve_serve.h"))
    return os.path.getmtime(SERVE_LIB) < max(os.path.getmtime(d) for d in deps)


def build_serve(force=False, verbose=True):
    os.makedirs(SERVE_BUILD, exist_ok=True)
    hdr = max(os.path.getmtime(os.path.join(SERVE_CSRC, f)) for f in os.listdir(SERVE_CSRC) if f.endswith(".h"))
    hdr = max(hdr, os.path.getmtime(os.path.join(os.path.dirname(HERE), "include", "qserve_serve.h")))

    def one(src):
        srcp, obj = os.path.join(SERVE_CSRC, src), os.path.join(SERVE_BUILD, src.replace(".hip", ".o"))
        if not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(srcp), hdr):
            return obj, False
        r = subprocess.run([hipcc(), *SERVE_FLAGS, "-c", srcp, "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
        return obj, True

    with cf.ThreadPoolExecutor(max_workers=min(8, len(SERVE_SOURCES))) as ex:
        res = list(ex.map(one, SERVE_SOURCES))
    if force or any(r for _, r in res) or not os.path.exists(SERVE_LIB):
        tmp = SERVE_LIB + f".tmp{os.getpid()}"           # (renamed into place: a process loading the library never sees half of it)
        r = subprocess.run([hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,--no-undefined", *[o for o, _ in res],
                            "-o", tmp], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
        os.replace(tmp, SERVE_LIB)
        if verbose:
            print(f"[qserve_amd.build] linked {SERVE_LIB}", file=sys.stderr)
    elif verbose:
        print(f"[qserve_amd.build] up to date: {SERVE_LIB}", file=sys.stderr)
    return SERVE_LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--serve", action="store_true", help="build only libqserve_serve.so (the paged serving engine's kernels)")
    ap.add_argument("--timing", action="store_true", help="build libqserve_amd_timing.so (-DQS_TIMING) instead")
    a = ap.parse_args()
    if a.serve:
        build_serve(force=a.force)
        sys.exit(0)
    build(force=a.force, timing=a.timing)
    build_serve(force=a.force)
    sys.exit(0)
