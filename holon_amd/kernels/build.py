"""Building libholon_hip.so from `holon_amd/csrc` with hipcc for gfx950.

The library is built in-tree (`holon_amd/kernels/libholon_hip.so`, objects under `holon_amd/csrc/_build`). When the
tree is not writable the build goes to a per-user folder under the system's temporary directory instead. A build
prints a line per file, so that a first call that has to compile does not look hung.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import pathlib
import shutil
import subprocess
import sys
import tempfile
import time

CSRC = pathlib.Path(__file__).resolve().parent.parent / "csrc"
IN_TREE = pathlib.Path(__file__).resolve().parent / "libholon_hip.so"
ARCH = "gfx950"
# Packed float32 VALU ops are kept out of the generated code on purpose. Matrix-core accumulators are kept in
# ordinary vector registers: with the accumulator file the compiler copies them back and forth around every
# rescale of the attention kernels (a third of their vector instructions).
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form=1", "-Wno-unused-command-line-argument"]


def sources() -> list[pathlib.Path]:
    return sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.cpp"))


def source_hash() -> str:
    h = hashlib.sha256()
    for f in sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.cpp")) + sorted(CSRC.glob("*.h")):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    h.update(" ".join(HIP_FLAGS).encode())
    return h.hexdigest()[:16]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and pathlib.Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc): the HIP kernels cannot be built")


def _writable(path: pathlib.Path) -> bool:
    try:
        path.mkdir(parents=True, exist_ok=True)
        probe = path / f".probe-{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def fallback_dir() -> pathlib.Path:
    return pathlib.Path(tempfile.gettempdir()) / f"holon_amd-{os.getuid()}" / source_hash()


def find_library() -> pathlib.Path | None:
    """The built library: in-tree first, then this source version's copy in the temporary folder."""
    if IN_TREE.is_file():
        return IN_TREE
    alt = fallback_dir() / "libholon_hip.so"
    return alt if alt.is_file() else None


def build(verbose: bool = True, force: bool = True) -> pathlib.Path:
    """Compile every source and link the library; returns its path."""
    say = (lambda m: print(f"holon_amd: {m}", file=sys.stderr, flush=True)) if verbose else (lambda m: None)
    if _writable(CSRC / "_build") and _writable(IN_TREE.parent):
        objdir, target = CSRC / "_build", IN_TREE
    else:
        objdir = fallback_dir()
        objdir.mkdir(parents=True, exist_ok=True)
        target = objdir / "libholon_hip.so"
    objdir = objdir / f"obj-{os.getpid()}"       # its own folder: two processes may build at the same time
    objdir.mkdir(parents=True, exist_ok=True)
    cc = hipcc()
    srcs = sources()
    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {target} (a minute or two the first time)")
    t0 = time.time()

    def compile_one(src: pathlib.Path) -> pathlib.Path:
        obj = objdir / (src.name + ".o")
        cmd = [cc, *HIP_FLAGS, "-c", str(src), "-o", str(obj)]
        if src.suffix == ".cpp":
            cmd = [cc, "-O2", "-std=c++17", "-fPIC", "-c", str(src), "-o", str(obj)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
        say(f"  compiled {src.name} ({time.time() - t0:.0f} s)")
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = target.parent / f"{target.name}.tmp{os.getpid()}"
    proc = subprocess.run([cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"linking libholon_hip.so failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, target)
    shutil.rmtree(objdir, ignore_errors=True)
    (target.parent / (target.name + ".hash")).write_text(source_hash())
    say(f"built {target} in {time.time() - t0:.0f} s")
    return target


def source_library(source: str | pathlib.Path) -> pathlib.Path | None:
    """The library built from one source file of a part's own (`lib<stem>.so` beside it, else in the per-user folder),
    if it is there and not older than the source."""
    source = pathlib.Path(source).resolve()
    for cand in (source.with_name(f"lib{source.stem}.so"), fallback_dir() / f"lib{source.stem}.so"):
        if cand.is_file() and cand.stat().st_mtime >= source.stat().st_mtime:
            return cand
    return None


def build_source(source: str | pathlib.Path, verbose: bool = True) -> pathlib.Path:
    """Compile one HIP source that a part brings with it into a library of its own, with this package's flags and
    headers (`holon_amd/csrc` is on the include path: `common.h` may be used)."""
    source = pathlib.Path(source).resolve()
    target = source.with_name(f"lib{source.stem}.so")
    if not _writable(target.parent):
        fallback_dir().mkdir(parents=True, exist_ok=True)
        target = fallback_dir() / target.name
    tmp = target.parent / f"{target.name}.tmp{os.getpid()}"
    t0 = time.time()
    proc = subprocess.run([hipcc(), *HIP_FLAGS, "-shared", f"-I{CSRC}", str(source), "-o", str(tmp)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {source}:\n{proc.stderr[-4000:]}")
    os.replace(tmp, target)
    if verbose:
        print(f"holon_amd: built {target} in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    return target


if __name__ == "__main__":
    build()
