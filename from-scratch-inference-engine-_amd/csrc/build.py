"""Builds the kernel library with hipcc for gfx950 and says where it is.

``build()`` always compiles.  ``ensure_built()`` compiles only when no library exists for the
present sources (first call in a fresh checkout) and prints a line per step so that a caller
waiting on it sees progress.  The library goes to ``csrc/_build/`` inside the checkout; if
that folder cannot be written (a read-only install), to a per-user folder under the system's
temporary directory.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
ARCH = "gfx950"
LIB_NAME = "libfsie_kernels.so"
# packed-fp32 code generation is switched off for every kernel of this library
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature",
               "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _say(msg: str) -> None:
    print(f"[fsie build] {msg}", file=sys.stderr, flush=True)


def sources():
    return sorted(CSRC.glob("*.hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found: the kernel library cannot be built "
                       "(set HIPCC or put /opt/rocm/bin on PATH)")


def _writable_dir(path: Path) -> bool:
    try:
        path.mkdir(parents=True, exist_ok=True)
        probe = path / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def private_tmp_dir(name: str):
    """``<tmp>/<name>-<uid>``, made with mode 0700 if it is not there; None unless it belongs to
    this user and nobody else may write to it.  The system's temporary folder is shared: a library
    or a file of results found in a folder that another user could have made or filled is not
    loaded."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    path = Path(tempfile.gettempdir()) / f"{name}-{uid}"
    try:
        path.mkdir(mode=0o700, exist_ok=True)
        st = path.lstat()
    except OSError:
        return None
    import stat

    if not stat.S_ISDIR(st.st_mode) or (hasattr(os, "getuid") and st.st_uid != uid) or (st.st_mode & 0o022):
        return None
    return path


def build_dirs():
    """Candidate folders, in the order they are looked at: the checkout's own, then a private
    per-user folder under the system's temporary directory."""
    dirs = [CSRC / "_build"]
    tmp = private_tmp_dir("fsie-build")
    if tmp is not None:
        dirs.append(tmp)
    return dirs


def find_built():
    """Path of a library built from the present sources, or None."""
    want = source_hash()
    for d in build_dirs():
        lib, stamp = d / LIB_NAME, d / "stamp"
        try:
            if lib.is_file() and stamp.is_file() and stamp.read_text().strip() == want:
                return lib
        except OSError:
            continue
    return None


def _compile_one(hipcc: str, src: Path, obj: Path):
    t0 = time.time()
    cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    return src, proc, time.time() - t0


def build(verbose: bool = True) -> Path:
    hipcc = _hipcc()
    out_dir = next((d for d in build_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library")
    srcs = sources()
    if verbose:
        _say(f"compiling {len(srcs)} sources for {ARCH} into {out_dir}")
    # objects go to a folder of this process, so that two first builds at once (a test run beside a
    # replay) do not write each other's files; only the finished library is moved into place
    obj_dir = out_dir / f"obj{os.getpid()}"
    obj_dir.mkdir(exist_ok=True)
    objs = [obj_dir / (s.stem + ".o") for s in srcs]
    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8"))))
    failed = []
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for src, proc, dt in pool.map(lambda so: _compile_one(hipcc, *so), zip(srcs, objs)):
            if proc.returncode != 0:
                failed.append((src, proc.stderr))
            elif verbose:
                _say(f"  {src.name} ({dt:.1f} s)")
    if failed:
        shutil.rmtree(obj_dir, ignore_errors=True)
        text = "\n".join(f"--- {s.name}\n{err}" for s, err in failed)
        raise RuntimeError(f"hipcc failed:\n{text}")
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    link = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)],
                          capture_output=True, text=True)
    shutil.rmtree(obj_dir, ignore_errors=True)
    if link.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{link.stderr}")
    os.replace(tmp, out_dir / LIB_NAME)
    (out_dir / "stamp").write_text(source_hash() + "\n")
    if verbose:
        _say(f"built {out_dir / LIB_NAME}")
    return out_dir / LIB_NAME


def ensure_built() -> Path:
    lib = find_built()
    if lib is not None:
        return lib
    _say("no kernel library for these sources yet: building once (a few seconds to half a minute, by the number of cores)")
    return build()


if __name__ == "__main__":
    print(build())
