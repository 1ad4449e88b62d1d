"""Build libmi355_hotpath.so (the C-ABI library of HIP kernels) in-tree with hipcc for gfx950.

hipcc cross-compiles without a GPU.  The .so is git-ignored but travels with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmi355_hotpath.so")
# the development build: the same sources with -DMI355_DEV_BUILD (ablation switches become run-time
# variables set through mi355_debug_set) plus the bandwidth probes; used by tools/, never by the package
LIB_DEV = os.path.join(HERE, "libmi355_hotpath_dev.so")
SOURCES = ["elementwise.hip", "index_ops.hip", "attn_decode.hip", "attn_extend.hip", "gemm.hip",
           "gemm_tiled.hip", "sampling.hip", "quant_fp8.hip", "allreduce.hip", "mla_proj.hip",
           "stream_ops.hip", "attn_latent.hip", "postnorm_ops.hip", "recurrence.hip", "attn_sigmoid.hip", "moe_ops.hip", "conv_ops.hip", "attn_window.hip"]
DEV_SOURCES = ["debug_bw.hip"]
HEADERS = [os.path.join(CSRC, "common.cuh"),
           os.path.join(os.path.dirname(HERE), "include", "mi355_hotpath.h"),
           os.path.join(os.path.dirname(HERE), "include", "mi355_hotpath_dev.h")]
# -amdgpu-mfma-vgpr-form: matrix-core accumulators stay in ordinary vector registers.  The kernels
# here run softmax / rescale / epilogue arithmetic on them between MFMAs; with the default AGPR
# form every such use costs a v_accvgpr_read/_write pair (hundreds per loop body in the attention
# kernels), and no kernel needs more than the 256 registers the VGPR form can address.
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-fno-gpu-rdc",
         "-Wno-unused-result", "-mllvm", "-amdgpu-mfma-vgpr-form",
         # no packed-fp32 instructions (v_pk_add/mul/fma_f32): the compiler forms them from ordinary float code by
         # itself otherwise; the host pass does not know the feature and says so, harmlessly
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


# What one model family needs of the library: a first call in a fresh checkout (bin/trace_run) compiles these and no
# more.  The result is a PARTIAL library at the usual path, marked by the file PARTIAL_MARK (one source name a line);
# entry points of the sources left out raise when called (_lib.load), and the next full build() completes it.
FAMILY_SOURCES = {
    "Seturax": ["elementwise.hip", "index_ops.hip", "gemm.hip", "gemm_tiled.hip", "stream_ops.hip", "attn_latent.hip"],
    "Verozen": ["elementwise.hip", "index_ops.hip", "gemm.hip", "gemm_tiled.hip", "postnorm_ops.hip", "recurrence.hip",
                "attn_sigmoid.hip", "moe_ops.hip"],
    "Gatarax": ["elementwise.hip", "index_ops.hip", "gemm.hip", "gemm_tiled.hip", "postnorm_ops.hip", "recurrence.hip",
                "moe_ops.hip", "conv_ops.hip", "attn_window.hip"],
    "Fudonex": ["elementwise.hip", "index_ops.hip", "gemm.hip", "gemm_tiled.hip", "postnorm_ops.hip", "recurrence.hip",
                "conv_ops.hip", "attn_window.hip"],
}
PARTIAL_MARK = LIB + ".partial"


def partial_sources():
    """Sources of the library at LIB if it is a partial build, else None."""
    if not (os.path.exists(LIB) and os.path.exists(PARTIAL_MARK)):
        return None
    with open(PARTIAL_MARK) as f:
        return [line.strip() for line in f if line.strip()]


def build_for(architecture: str, verbose: bool = False) -> str:
    """The library as far as `architecture` needs it: a complete library is kept complete (used as it is, or rebuilt
    whole if a source is newer); where there is none, or a partial one, the family's sources alone are built
    (everything, for a family without a list)."""
    only = FAMILY_SOURCES.get(architecture)
    if only is None:
        return build(verbose=verbose)
    have = partial_sources()
    if os.path.exists(LIB) and have is None:
        # a complete library is never replaced by a partial one: it is used, or, if a source is newer, rebuilt whole
        return build(verbose=verbose)
    if have is not None:
        only = sorted(set(only) | set(have))
    return build(verbose=verbose, only=only)


def build(force: bool = False, verbose: bool = False, dev: bool = False, only=None) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build_dev" if dev else "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES + (DEV_SOURCES if dev else []) if os.path.exists(os.path.join(CSRC, s))]
    if only is not None:
        assert not dev
        srcs = [s for s in srcs if s in set(only)]
        if len(srcs) == len(SOURCES):
            only = None
    lib = LIB_DEV if dev else LIB
    if not dev and only is None and os.path.exists(PARTIAL_MARK):
        force_link = True        # a partial library is at the path: link again whatever the time stamps say
    else:
        force_link = False
    flags = FLAGS + (["-DMI355_DEV_BUILD"] + os.environ.get("MI355_DEV_EXTRA_FLAGS", "").split() if dev else [])
    objs, procs = [], []
    for s in srcs:
        src = os.path.join(CSRC, s)
        obj = os.path.join(objdir, s.replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, [src] + HEADERS):
            cmd = [hipcc] + flags + ["-c", src, "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for s, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- hipcc failed on {s} ---\n{out.decode()}\n")
    if failed:
        raise RuntimeError("hipcc compilation failed")
    was_partial = partial_sources() if not dev else None
    if only is not None and (was_partial is None or set(was_partial) != set(srcs)):
        force_link = True
    if force or procs or force_link or _stale(lib, objs):
        cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    if not dev:
        if only is not None:
            with open(PARTIAL_MARK, "w") as f:
                f.write("\n".join(srcs) + "\n")
        elif os.path.exists(PARTIAL_MARK):
            os.remove(PARTIAL_MARK)
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True, dev="--dev" in sys.argv))
