"""Compiles the HIP sources of this package for gfx950 into elmo_amd/libelmo_xmc.so (in-tree)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "xmc_capi.hip")
OUT = os.path.join(HERE, "libelmo_xmc.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


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
    cmd = [hipcc] + HIPCC_FLAGS + [f'-DXMC_SOURCE_HASH="{digest}"', SRC, "-o", tmp]
    if verbose:
        cmd.append("-Rpass-analysis=kernel-resource-usage")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
    # moved into place in one step: a process that has the previous library mapped keeps its (unlinked) file
    os.replace(tmp, OUT)
    with open(HASH_FILE, "w") as f:
        f.write(digest + "\n")
    return res.stderr if verbose else OUT


def ensure_built():
    """Builds the library only if none is there (tests, the smoke run and the benchmark load what is built)."""
    return OUT if os.path.exists(OUT) else build()


if __name__ == "__main__":
    print(build(verbose=True))
