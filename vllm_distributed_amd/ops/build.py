"""Build the native libraries in-tree with hipcc for gfx950 (cross-compiles
without a GPU).

    python -m vllm_distributed_amd.ops.build [--force] [--jobs N]

Produces, next to this file:
    libvda_ops.so    HIP kernels of ops/csrc/*.hip (C ABI, loaded with ctypes)
    libvda_comm.so   peer-memory collectives of parallel/csrc
    libvda_host.so   host-only runtime of runtime/csrc (g++): shared-memory RPC ring
Object files and content hashes live in ops/build/ so unchanged sources are
not recompiled.
"""
from __future__ import annotations

import argparse
import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
ARCH = "gfx950"

LIBS = {
    "libvda_ops.so": {
        "dir": os.path.join(HERE, "csrc"),
        "out": os.path.join(HERE, "libvda_ops.so"),
        "ldflags": [],
    },
    "libvda_comm.so": {
        "dir": os.path.join(PKG, "parallel", "csrc"),
        "out": os.path.join(PKG, "parallel", "libvda_comm.so"),
        "ldflags": ["-lpthread", "-lrt"],
    },
    # host-only runtime (no device code): shared-memory RPC ring, block hashing
    "libvda_host.so": {
        "dir": os.path.join(PKG, "runtime", "csrc"),
        "out": os.path.join(PKG, "runtime", "libvda_host.so"),
        "ldflags": ["-lpthread", "-lrt"],
        "host": True,
    },
}


# Per-file additions to the device flags.  The online-softmax kernels keep their MFMA accumulators in
# ordinary VGPRs: with the accumulator-register form the compiler copied every output register out and
# back around the conditional rescale (attention.hip: ~130 of ~470 vector instructions per key tile;
# mla.hip: 3296 accumulator moves in six kernels, 400 -> 269 registers).  Measured neutral on the
# memory-bound skinny GEMMs, which therefore keep the default.
_VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
EXTRA_FLAGS = {f: _VGPR_FORM for f in ("attention.hip", "attention_prefill.hip", "mla.hip")}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _digest(path: str, extra: str) -> str:
    h = hashlib.sha256(extra.encode())
    d = os.path.dirname(path)
    for p in [path] + sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".h")):
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _compile_one(src: str, obj: str, flags: list[str], force: bool, cc: str | None = None) -> tuple[str, bool]:
    stamp = obj + ".sha"
    want = _digest(src, " ".join(flags))
    if not force and os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == want:
        return src, False
    cmd = [cc or _hipcc(), *flags, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    with open(stamp, "w") as f:
        f.write(want)
    return src, True


# kernels every generation path launches (linear layers, gated activations, norms, sampling); a model class adds its
# own in ``native_sources``
COMMON_OPS_SOURCES = ("activation.hip", "norm.hip", "sampling.hip", "gemm_dense.hip", "gemv.hip", "gemm_decode.hip")


def ensure_built_for(model_dir: str | None, log=None) -> None:
    """Build what a fresh checkout lacks before the engine starts.  When the model's class lists the kernel files
    it launches (``native_sources``), only those and the common ones are compiled into libvda_ops.so (a later full
    build adds the rest); otherwise everything is."""
    out = log or sys.stderr
    have = all(os.path.exists(spec["out"]) for name, spec in LIBS.items() if name != "libvda_comm.so")
    if have:
        return
    only = None
    try:
        from ..config import load_hf_config
        from ..models.registry import ModelRegistry
        cls, _ = ModelRegistry.resolve_model_cls(list(load_hf_config(model_dir).get("architectures") or []))
        extra = getattr(cls, "native_sources", None)
        if extra is not None:
            only = tuple(COMMON_OPS_SOURCES) + tuple(extra)
    except Exception as e:       # unknown model: build everything, the engine will say what is wrong with it
        print(f"[build] model not recognised before the build ({type(e).__name__}): building all kernels", file=out,
              flush=True)
    print(f"[build] native libraries missing: compiling {'all kernels' if only is None else ', '.join(only)}",
          file=out, flush=True)
    build(verbose=False, only=only, skip=("libvda_comm.so",) if only is not None else ())
    print("[build] done", file=out, flush=True)


def build(force: bool = False, jobs: int | None = None, verbose: bool = True, only: tuple | None = None,
          skip: tuple = ()) -> list[str]:
    """``only``: file names of ops/csrc to put into libvda_ops.so (None: all of them)."""
    jobs = jobs or min(16, os.cpu_count() or 1)
    flags = [f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-ffast-math", "-fno-finite-math-only",
             "-fvisibility=hidden", "-Wno-unused-value", "-DNDEBUG",
             # no packed fp32 arithmetic: the compiler forms v_pk_*_f32 from plain float code by itself
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    built = []
    for name, spec in LIBS.items():
        srcdir = spec["dir"]
        if not os.path.isdir(srcdir) or name in skip:
            continue
        srcs = sorted(os.path.join(srcdir, f) for f in os.listdir(srcdir) if f.endswith((".hip", ".cpp")))
        if only is not None and name == "libvda_ops.so":
            srcs = [p_ for p_ in srcs if os.path.basename(p_) in only]
        if not srcs:
            continue
        objdir = os.path.join(HERE, "build", name.split(".")[0])
        os.makedirs(objdir, exist_ok=True)
        objs = [os.path.join(objdir, os.path.basename(s) + ".o") for s in srcs]
        changed = False
        host = spec.get("host", False)
        cc = (shutil.which("g++") or "g++") if host else None
        fl = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-DNDEBUG"] if host else flags
        with ThreadPoolExecutor(jobs) as ex:
            for src, did in ex.map(lambda a: _compile_one(a[0], a[1], fl + ([] if host else EXTRA_FLAGS.get(
                    os.path.basename(a[0]), [])), force, cc), zip(srcs, objs)):
                changed |= did
                if verbose and did:
                    print(f"[build] compiled {os.path.relpath(src, PKG)}", flush=True)
        out = spec["out"]
        # a library linked from a subset of the sources is completed by the next full build
        listing = os.path.join(objdir, "linked.txt")
        linked = open(listing).read().split() if os.path.exists(listing) else None
        want = sorted(os.path.basename(o) for o in objs)
        if changed or not os.path.exists(out) or (linked is not None and linked != want):
            cmd = [cc, "-shared", "-fPIC", "-o", out, *objs, *spec["ldflags"]] if host else \
                [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", out, *objs, *spec["ldflags"]]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"link failed for {name}:\n{r.stdout}\n{r.stderr}")
            with open(listing, "w") as f:
                f.write("\n".join(want))
            if verbose:
                print(f"[build] linked {os.path.relpath(out, PKG)}", flush=True)
        built.append(out)
    return built


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=None)
    a = ap.parse_args()
    for p in build(a.force, a.jobs):
        print(p)
