"""Build the gfx950 C-ABI shared library in-tree with hipcc (no torch extension machinery).

    python -m lite_llama_amd.build          # -> lite_llama_amd/lib/liblite_llama_amd.so

hipcc cross-compiles for gfx950 without a GPU; the built .so is git-ignored but travels
to the GPU box with the repo snapshot.
"""

from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "liblite_llama_amd.so"
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off"]
FLAGS += os.environ.get("LL_EXTRA_HIPCC_FLAGS", "").split()  # debug builds (e.g. -DV2_DEBUG_ABLATE)
# per-source flags.  gemm_short.hip: its kernel's first 16 argument dwords arrive in SGPRs with the wave (gfx950 kernarg preload)
# instead of through dependent scalar loads -- a launch of ~5 us spends ~0.3 us there otherwise.
# seq_mix.hip / ragged_attn*.hip: no packed fp32 arithmetic made from ordinary float code (the host pass warns that it does not
# know the feature).  The older sources keep the flags their bit-exactness tests were pinned under: with the feature off, two
# norm kernels that must agree bit for bit (rows summed over MoE slots vs. summed first) select different roundings.
_NO_PACKED_FP32 = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FILE_FLAGS = {"gemm_short.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
              "seq_mix.hip": _NO_PACKED_FP32, "ragged_attn.hip": _NO_PACKED_FP32, "ragged_attn_mfma.hip": _NO_PACKED_FP32,
              "group_norm.hip": _NO_PACKED_FP32, "latent_attn.hip": _NO_PACKED_FP32, "moe_sparse.hip": _NO_PACKED_FP32,
              "linear_mix.hip": _NO_PACKED_FP32}


# part libraries: the sources ONE model family needs (a fresh checkout serving only that family builds nothing else)
PARTS = {"ragged": ["seq_mix.hip", "ragged_attn.hip", "ragged_attn_mfma.hip", "group_norm.hip", "latent_attn.hip", "moe_sparse.hip",
                    "linear_mix.hip", "kv_paged.hip", "kv_ops.hip", "sampler.hip"]}


def flags_for(src: str) -> list[str]:
    return FLAGS + FILE_FLAGS.get(os.path.basename(src), [])


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (expected /opt/rocm/bin/hipcc)")


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _digest(paths: list[str]) -> str:
    h = hashlib.sha256()
    headers = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))
    for p in sorted(paths) + headers + [os.path.join(HERE, "..", "include", "lite_llama_amd.h")]:
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()


def lib_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


def part_path(part: str) -> str:
    return os.path.join(LIBDIR, f"liblite_llama_amd_{part}.so")


def ensure(part: str, verbose: bool = False) -> str:
    """What a model family's entry point calls first: the full library if it is built and current, else the family's part
    library, compiled now if it is missing or stale."""
    stamp = os.path.join(LIBDIR, "build.stamp")
    if os.path.exists(lib_path()) and os.path.exists(stamp) and open(stamp).read().strip() == _digest(sources()):
        return lib_path()
    return build(verbose=verbose, part=part)


def build(force: bool = False, verbose: bool = True, part: str | None = None) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sources() if part is None else [os.path.join(CSRC, f) for f in PARTS[part]]
    target = lib_path() if part is None else part_path(part)
    stamp = os.path.join(LIBDIR, "build.stamp" if part is None else f"build_{part}.stamp")
    digest = _digest(srcs)
    if not force and os.path.exists(target) and os.path.exists(stamp):
        if open(stamp).read().strip() == digest:
            return target
    hipcc = _hipcc()
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        one = _digest([src]) + " " + " ".join(flags_for(src))  # (covers the headers too)
        if not force and os.path.exists(obj) and os.path.exists(obj + ".stamp") and open(obj + ".stamp").read() == one:
            return obj  # an object of exactly this source, headers and flags is there
        cmd = [hipcc, *flags_for(src), "-c", src, "-o", obj]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        done = subprocess.run(cmd, stderr=None if verbose else subprocess.PIPE, text=True)
        if done.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{done.stderr or ''}")
        with open(obj + ".stamp", "w") as f:
            f.write(one)
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(compile_one, srcs))
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", target + ".tmp"]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    os.replace(target + ".tmp", target)
    with open(stamp, "w") as f:
        f.write(digest)
    return target


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
