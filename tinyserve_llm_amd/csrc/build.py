"""Compiles the HIP sources of this folder for gfx950 into one shared library with hipcc.

No torch headers and no ninja are involved: every kernel has an `extern "C"` launcher that takes
raw device pointers and a stream, and Python calls them through ctypes. The library is written next
to the sources; if that folder is read-only, to a per-user folder under the system's temporary
directory (made with mode 0700, and used only if it is this user's own and closed to everyone else). A sidecar file records a hash of the sources and flags so that a stale library is
rebuilt and a current one is loaded as it is.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libtinyserve_hip.so"
ARCH = "gfx950"
FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
    # packed 32-bit float instructions are switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results stay in ordinary vector registers: the softmax and the epilogues work on
    # them with vector instructions, and copies to and from the accumulation registers cost more
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    # the first kernel arguments arrive in scalar registers with the wave instead of being loaded
    # by its first instructions: a decode step is a hundred short kernels, each of which would
    # otherwise start with a trip to memory for its arguments
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


# the vendor's matrix library, which gemm_library.hip calls for products with many rows
LINK = ["-lhipblaslt"]


def sources() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + LINK).encode())
    for name in sorted(f for f in os.listdir(HERE) if f.endswith((".hip", ".h"))):
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                       "the HIP kernels cannot be built and there is no other path")


def _private(folder: str) -> bool:
    """Whether a folder outside the package is this user's alone: a real directory (no link) that
    the user owns and nobody else may write to. The temporary directory is shared, its per-user
    folder has a name anyone can guess, and a library found there is loaded into the process: a
    folder that someone else made, or may write into, is not used."""
    try:
        st = os.lstat(folder)
    except OSError:
        return False
    import stat
    return stat.S_ISDIR(st.st_mode) and st.st_uid == os.getuid() and not st.st_mode & 0o022


def _usable(folder: str, create: bool) -> bool:
    """Whether the library may be read from (and, with `create`, written to) `folder`."""
    if folder != HERE:
        if create and not os.path.lexists(folder):
            try:
                os.mkdir(folder, 0o700)
            except OSError:
                return False
        if not _private(folder):
            return False
    if not create:
        return os.path.isdir(folder)
    try:
        probe = os.path.join(folder, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def candidate_dirs() -> list[str]:
    return [HERE, os.path.join(tempfile.gettempdir(), f"tinyserve_llm_amd_{os.getuid()}")]


def find_current() -> str | None:
    """Path of a built library whose recorded hash matches the sources, or None."""
    want = source_hash()
    for folder in candidate_dirs():
        if not _usable(folder, create=False):
            continue
        lib, stamp = os.path.join(folder, LIB_NAME), os.path.join(folder, LIB_NAME + ".hash")
        try:
            with open(stamp) as f:
                if f.read().strip() == want and os.path.exists(lib):
                    return lib
        except OSError:
            continue
    return None


def build(verbose: bool = True, force: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    if not force:
        lib = find_current()
        if lib:
            return lib
    hipcc = _hipcc()
    out_dir = next((d for d in candidate_dirs() if _usable(d, create=True)), None)
    if out_dir is None:
        raise RuntimeError(f"no folder for the kernel library among {candidate_dirs()}: each is read-only, or is not "
                           "this user's own (owned by someone else, or writable by others)")
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)  # hipcc wants a home for its caches; an empty HOME is fine
    if not env.get("HOME"):
        env["HOME"] = out_dir
    srcs = sources()
    say = (lambda msg: print(f"[tinyserve_llm_amd build] {msg}", file=sys.stderr, flush=True)) if verbose else (lambda msg: None)
    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    start = time.time()
    errors: list[str] = []
    objs = [os.path.join(obj_dir, s[:-4] + ".o") for s in srcs]

    def compile_one(src: str, obj: str) -> None:
        cmd = [hipcc, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode:
            errors.append(f"{' '.join(cmd)}\n{r.stdout}{r.stderr}")
        else:
            say(f"compiled {src} ({time.time() - start:.0f} s)")

    threads = [threading.Thread(target=compile_one, args=(s, o)) for s, o in zip(srcs, objs)]
    for t in threads:
        t.start()
    while any(t.is_alive() for t in threads):
        for t in threads:
            t.join(timeout=10.0 / len(threads))
        if any(t.is_alive() for t in threads) and int(time.time() - start) % 10 == 0:
            say(f"still compiling ({time.time() - start:.0f} s)")
            time.sleep(1.0)
    if errors:
        raise RuntimeError("hipcc failed:\n" + "\n".join(errors))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, *LINK, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if r.returncode:
        raise RuntimeError(f"link failed: {' '.join(cmd)}\n{r.stdout}{r.stderr}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash())
    say(f"built {lib} in {time.time() - start:.0f} s")
    return lib


if __name__ == "__main__":
    print(build())
