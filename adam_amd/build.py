"""Build libadamah_hip.so (gfx950) in-tree with hipcc: `python -m adam_amd.build`."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libadamah_hip.so")
SOURCES = ["runtime.hip", "gemv_q.hip", "gemv_mfma.hip", "gemm_q4_mfma.hip", "fuse.hip", "norm_rope.hip", "rowprep.hip", "attention.hip", "attn_decode.hip", "attn_prefill.hip", "elementwise.hip", "sampling.hip", "topk_fused.hip", "fused_proj.hip", "token_feed.hip", "probe.hip"]
# -amdgpu-kernarg-preload-count: the first 14 dwords of a kernel's arguments (whole scalars / pointers, in order) are
# in SGPRs when a wave starts instead of being fetched from the argument block -- one trip to memory less before a
# kernel's first loads (Q4 GEMV 5.8 -> 5.4 us at 4096x4096).  The hot kernels order their arguments for it.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=14",
         "-Wno-unused-result", "-Wno-unused-value"]
# gemv_mfma.hip draws a ticket with one atomic per workgroup and looks at it much later; the
# compiler's wave-level aggregation of uniform-address atomics would wait for the result at once.
# attn_prefill.hip: the matrix instructions' results in ordinary vector registers.  With the accumulator registers the
# compiler otherwise picks, the chunk attention's 32 running output values moved to vector registers and back in every
# key tile (64 of ~300 vector instructions per tile) because the score products wanted the same accumulator registers.
EXTRA = {"gemv_mfma.hip": ["-mllvm", "-amdgpu-atomic-optimizer-strategy=None"],
         "attn_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    return "hipcc"


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in p.stdout.splitlines() if noise not in l)
    if p.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{out}")
    return out


def build(verbose=True, jobs=None):
    """Compile every source for gfx950 and link the shared library next to this package."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def one(i):
        return _run([hipcc, *FLAGS, *EXTRA.get(SOURCES[i], []), "-c", os.path.join(CSRC, SOURCES[i]), "-o", objs[i]])

    with ThreadPoolExecutor(max_workers=jobs or min(len(SOURCES), os.cpu_count() or 4)) as ex:
        for s, out in zip(SOURCES, ex.map(one, range(len(SOURCES)))):
            if verbose and out.strip():
                print(f"[{s}]\n{out}")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", OUT])
    if verbose:
        print(f"built {OUT} ({os.path.getsize(OUT) // 1024} KiB)")
    return OUT


if __name__ == "__main__":
    try:
        build()
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
