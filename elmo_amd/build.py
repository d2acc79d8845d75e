"""Compiles the HIP sources of this package for gfx950 into elmo_amd/libelmo_xmc.so (in-tree)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "xmc_capi.hip")
OUT = os.path.join(HERE, "libelmo_xmc.so")

SRC_HEAVY = os.path.join(HERE, "csrc", "xmc_fp8_role_heavy.hip")
SRC_PLAIN = os.path.join(HERE, "csrc", "xmc_fp8_role_plain.hip")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# The second translation unit holds the variants of the step kernel whose tile loop is too large for the compiler's
# default "#pragma unroll" size limit (see the head of that file); everything else keeps the default.  The scheduler
# settings are those of the third unit: with them the Philox variant spills 7 registers instead of 39 (0.92 against
# 1.11 ms per launch) and the head-Kahan ones 15 instead of 26.
HEAVY_FLAGS = ["-mllvm", "-pragma-unroll-threshold=1000000", "-mllvm", "-misched-cluster=0", "-mllvm", "-amdgpu-use-amdgpu-trackers=1"]
# The third one holds the headline variants of the step kernel, with the instruction scheduler settings that measured
# best for them (see the head of that file).
PLAIN_FLAGS = ["-mllvm", "-misched-cluster=0", "-mllvm", "-amdgpu-use-amdgpu-trackers=1"]


def source_files():
    csrc = os.path.join(HERE, "csrc")
    return sorted(os.path.join(csrc, f) for f in os.listdir(csrc)) + [os.path.join(os.path.dirname(HERE), "include", "elmo_xmc.h")]


def source_hash():
    """Digest of the HIP sources and the header; the library reports the one it was built from (xmc_source_hash)."""
    import hashlib
    h = hashlib.sha256()
    for path in source_files():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


HASH_FILE = OUT + ".hash"


def built_hash():
    """Digest of the sources the library in the tree was built from (written by build()), or None."""
    try:
        with open(HASH_FILE) as f:
            return f.read().strip()
    except OSError:
        return None


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    digest = source_hash()
    tmp = OUT + ".tmp%d" % os.getpid()
    extra = ["-Rpass-analysis=kernel-resource-usage"] if verbose else []
    objs = [tmp + ".main.o", tmp + ".heavy.o", tmp + ".plain.o"]
    cmds = [[hipcc] + HIPCC_FLAGS + extra + [f'-DXMC_SOURCE_HASH="{digest}"', "-c", SRC, "-o", objs[0]],
            [hipcc] + HIPCC_FLAGS + HEAVY_FLAGS + extra + ["-c", SRC_HEAVY, "-o", objs[1]],
            [hipcc] + HIPCC_FLAGS + PLAIN_FLAGS + extra + ["-c", SRC_PLAIN, "-o", objs[2]]]
    procs = [subprocess.Popen(c, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True) for c in cmds]   # side by side
    outs = [p.communicate() for p in procs]
    log = "".join(o[0] + o[1] for o in outs)
    try:
        if any(p.returncode != 0 for p in procs):
            raise RuntimeError("hipcc failed:\n" + log)
        res = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", tmp], capture_output=True, text=True)
        if res.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            raise RuntimeError("hipcc (link) failed:\n" + res.stdout + res.stderr)
    finally:
        for o in objs:
            if os.path.exists(o):
                os.remove(o)
    # moved into place in one step: a process that has the previous library mapped keeps its (unlinked) file
    os.replace(tmp, OUT)
    with open(HASH_FILE, "w") as f:
        f.write(digest + "\n")
    return log if verbose else OUT


def ensure_built():
    """Builds the library only if none is there (tests, the smoke run and the benchmark load what is built)."""
    return OUT if os.path.exists(OUT) else build()


if __name__ == "__main__":
    print(build(verbose=True))
