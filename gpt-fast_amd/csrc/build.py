"""Compiling the HIP sources of this folder for gfx950 into shared libraries.

Each ``<name>.hip`` becomes ``build/libgfa_<name>.so`` (plain ``hipcc -shared``, C entry
points, no Python headers) with a stamp file beside it that holds a hash of what it was
built from (the source, the headers of this folder, the flags).  ``ensure(names)`` compiles the libraries
that are asked for and are missing or whose stamp no longer fits the sources, so an edited
kernel is never run from an old library; ``build_all()`` compiles every one anew.  Nothing
here needs a GPU: hipcc cross-compiles.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

HERE = os.path.dirname(os.path.abspath(__file__))
MODULES = ("core", "sampling", "gemm_bf16", "gemm_wide_bf16", "gemm_tiled_bf16", "attention_bf16",
           "ceilings")
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result", "-mllvm", "-amdgpu-kernarg-preload-count=16"]


class BuildError(RuntimeError):
    pass


def available_modules():
    return tuple(m for m in MODULES if os.path.isfile(os.path.join(HERE, m + ".hip")))


def _build_dir() -> str:
    """``build/`` beside the sources if it can be written, else a per-user folder under
    the temporary directory."""
    d = os.path.join(HERE, "build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"gfa_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def source_hash(name: str) -> str:
    """Hash of everything the library of module ``name`` is built from."""
    h = hashlib.sha256()
    headers = sorted(f for f in os.listdir(HERE) if f.endswith(".h"))
    for path in [os.path.join(HERE, name + ".hip")] + [os.path.join(HERE, h) for h in headers]:
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _is_current(path: str, name: str) -> bool:
    """The library at ``path`` exists and was built from the sources as they are now."""
    if not os.path.isfile(path):
        return False
    try:
        with open(path + ".stamp") as f:
            return f.read().strip() == source_hash(name)
    except OSError:
        return False


def _candidates(name: str):
    yield os.path.join(HERE, "build", f"libgfa_{name}.so")
    yield os.path.join(tempfile.gettempdir(), f"gfa_build_{os.getuid()}", f"libgfa_{name}.so")


def library_path(name: str) -> str:
    """Where the current library of module ``name`` is, or would be put."""
    for path in _candidates(name):
        if _is_current(path, name):
            return path
    return os.path.join(_build_dir(), f"libgfa_{name}.so")


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels of this library cannot be built")


def _compile(name: str, out: str, log) -> None:
    src = os.path.join(HERE, name + ".hip")
    stamp = source_hash(name)                         # of the sources as they are compiled
    tmp = out + f".tmp{os.getpid()}"
    cmd = [_hipcc()] + FLAGS + ["-I", HERE, src, "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())     # hipcc wants a writable home
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env,
                            cwd=os.path.dirname(out))
    done = threading.Event()

    def progress():
        t0 = time.time()
        while not done.wait(15.0):
            log(f"[gpt_fast_amd] still compiling {name}.hip ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=progress, daemon=True)
    th.start()
    output = proc.communicate()[0].decode("utf-8", "replace")
    done.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"hipcc failed on {name}.hip:\n{output}")
    os.replace(tmp, out)
    with open(out + ".stamp.tmp", "w") as f:
        f.write(stamp)
    os.replace(out + ".stamp.tmp", out + ".stamp")


def build(names, force=False, log=None) -> None:
    log = log or (lambda s: print(s, file=sys.stderr, flush=True))
    todo = []
    for n in names:
        if n not in available_modules():
            raise BuildError(f"no source {n}.hip in {HERE}")
        if force or not _is_current(library_path(n), n):
            todo.append((n, os.path.join(_build_dir(), f"libgfa_{n}.so")))
    if not todo:
        return
    log(f"[gpt_fast_amd] compiling {', '.join(n for n, _ in todo)} for {ARCH} ...")
    t0 = time.time()
    errors = []

    def work(item):
        try:
            _compile(item[0], item[1], log)
        except Exception as e:       # collected, raised below
            errors.append(e)
    threads = [threading.Thread(target=work, args=(it,)) for it in todo]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    log(f"[gpt_fast_amd] compiled in {time.time() - t0:.0f} s")


def ensure(names) -> None:
    """Build the named libraries that are missing or older than their sources."""
    build(names, force=False)


def build_all() -> None:
    build(available_modules(), force=True)


if __name__ == "__main__":
    build_all()
