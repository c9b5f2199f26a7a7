"""Builds libncn_hip.so (the C-ABI HIP library) in-tree with hipcc for gfx950.

The library has no PyTorch or Python dependency (plain C ABI, see include/ncn_hip.h), so it is
compiled by calling hipcc directly, one translation unit per process, and linked into
ncn_cuda_amd/libncn_hip.so.  hipcc cross-compiles without a GPU.

What is stale is decided by content, never by file times: every object file is kept with the hash of what it was
made from (its source, every header, its flags), and the library carries the hash of all of them
(`ncn_build_id()`, compiled into csrc/ncn_build_id.hip), which the loader compares with the sources it finds.
"""
import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libncn_hip.so")
BUILD_DIR = os.path.join(PKG_DIR, "build")
LOCK_PATH = os.path.join(PKG_DIR, ".build.lock")
ID_SOURCE = "ncn_build_id.hip"
SOURCES = ["ncn_api.hip", "ncn_fwd.hip", "ncn_bwd.hip", "ncn_bwd_once.hip", "ncn_fwd_indexed.hip", "ncn_bwd_indexed.hip", "ncn_bwd_indexed_once.hip",
           "ncn_headwise.hip", "ncn_headwise_indexed.hip", "ncn_headwise_bwd.hip", "ncn_headwise_bwd_indexed.hip", "ncn_generic.hip", "ncn_fused.hip", "ncn_fused_radix.hip", "ncn_fused_lengths.hip", "ncn_fused_headwise.hip", "ncn_fused_headwise_lengths.hip",
           "ncn_fused_radix_headwise.hip", "ncn_probe.hip", ID_SOURCE]
# packed-fp32 VALU instructions are switched off for device code on purpose (flag is device-only;
# the host pass prints a harmless "not a recognized feature" note).
HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
ID_MARKER = "NCN_BUILD_ID="    # the library holds this marker followed by the 16 hex digits of its build id


# Instruction scheduling per translation unit.  The multi-stage kernels wait on latency (LDS, barriers, dependent
# chains of two-row tiles): LLVM's max-ILP strategy measured 2.5 % on the 13-stage configuration, 1.5 % on the
# one-stage forward and 1.2 % on a step through the table builds; the plain one-stage backward with its loop over
# tiles is bound by issue slots and does not care, its form without the loop gains 2.5 % at 16 rows per group.
MAX_ILP = ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]
EXTRA_FLAGS = {"ncn_fused.hip": MAX_ILP, "ncn_fused_radix.hip": MAX_ILP, "ncn_fused_lengths.hip": MAX_ILP,
               "ncn_fused_headwise.hip": MAX_ILP, "ncn_fused_headwise_lengths.hip": MAX_ILP,
               "ncn_fused_radix_headwise.hip": MAX_ILP,
               "ncn_fwd.hip": MAX_ILP, "ncn_fwd_indexed.hip": MAX_ILP, "ncn_bwd_indexed.hip": MAX_ILP,
               "ncn_bwd_once.hip": MAX_ILP, "ncn_bwd_indexed_once.hip": MAX_ILP,
               "ncn_headwise.hip": MAX_ILP, "ncn_headwise_indexed.hip": MAX_ILP, "ncn_headwise_bwd.hip": MAX_ILP,
               "ncn_headwise_bwd_indexed.hip": MAX_ILP}


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: cannot build libncn_hip.so")
    return exe


def have_hipcc():
    return os.path.exists(shutil.which("hipcc") or "/opt/rocm/bin/hipcc")


def have_sources():
    return os.path.isdir(CSRC) and os.path.isdir(INCLUDE) and all(os.path.exists(os.path.join(CSRC, s)) for s in SOURCES)


def _read(path):
    with open(path, "rb") as fh:
        return fh.read()


def _headers_digest():
    """One hash over every header a translation unit can include (they are few and small: no per-unit dependency scan)."""
    h = hashlib.sha256()
    for root in (CSRC, INCLUDE):
        for name in sorted(os.listdir(root)):
            if name.endswith(".h"):
                h.update(name.encode() + b"\0" + _read(os.path.join(root, name)) + b"\0")
    return h.digest()


def unit_hash(src, headers=None):
    """Hash of everything the object file of `src` is made from, except the build id itself."""
    h = hashlib.sha256()
    h.update(headers if headers is not None else _headers_digest())
    h.update(" ".join(HIPCC_FLAGS + EXTRA_FLAGS.get(src, [])).encode() + b"\0")
    h.update(_read(os.path.join(CSRC, src)))
    return h.hexdigest()


def source_build_id():
    """The build id a library made from the sources as they are now would carry: 16 hex digits."""
    headers = _headers_digest()
    h = hashlib.sha256()
    for src in SOURCES:
        h.update(src.encode() + b"\0" + unit_hash(src, headers).encode() + b"\0")
    return h.hexdigest()[:16]


def library_build_id(path=LIB_PATH):
    """The build id compiled into the library file at `path` (read from the file, nothing is loaded), or None."""
    try:
        data = _read(path)
    except OSError:
        return None
    k = data.find(ID_MARKER.encode())
    if k < 0:
        return None
    digits = data[k + len(ID_MARKER):k + len(ID_MARKER) + 16]
    try:
        text = digits.decode("ascii")
        int(text, 16)
    except (UnicodeDecodeError, ValueError):
        return None
    return text if len(text) == 16 else None


def _compile(args):
    src, obj, want, build_id = args
    tmp = f"{obj}.{os.getpid()}.tmp"
    defs = [f'-DNCN_BUILD_ID_TEXT="{ID_MARKER}{build_id}"'] if src == ID_SOURCE else []
    cmd = [_hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), *defs, "-c", os.path.join(CSRC, src), "-o", tmp]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.unlink(tmp)
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, obj)
    with open(obj + ".hash", "w") as fh:
        fh.write(want)
    return src


def _object_is_current(obj, want):
    try:
        with open(obj + ".hash") as fh:
            return os.path.exists(obj) and fh.read().strip() == want
    except OSError:
        return False


def build(verbose=False, force=True):
    """Compile and link the shared library; returns the list of translation units that were compiled.

    force=True recompiles every unit.  force=False recompiles the units whose source, headers or flags differ in
    content from what their object file was made from, and links only if something was compiled or the library's build
    id is not that of the sources.  One build at a time per checkout (file lock); temporary files carry the process id.
    """
    os.makedirs(BUILD_DIR, exist_ok=True)
    with open(LOCK_PATH, "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            build_id = source_build_id()
            if not force and library_build_id() == build_id:
                return []                      # another process built it while this one waited for the lock
            headers = _headers_digest()
            jobs, objs = [], []
            for s in SOURCES:
                obj = os.path.join(BUILD_DIR, s.replace(".hip", ".o"))
                want = unit_hash(s, headers) + (build_id if s == ID_SOURCE else "")
                objs.append(obj)
                if force or not _object_is_current(obj, want):
                    jobs.append((s, obj, want, build_id))
            with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as pool:
                compiled = list(pool.map(_compile, jobs))
            tmp = f"{LIB_PATH}.{os.getpid()}.tmp"
            cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
            proc = subprocess.run(cmd, capture_output=True, text=True)
            if proc.returncode != 0:
                raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
            os.replace(tmp, LIB_PATH)
            if verbose:
                print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes, build id {build_id}, "
                      f"{len(compiled)} of {len(SOURCES)} units compiled)", file=sys.stderr)
            return compiled
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)


if __name__ == "__main__":
    build(verbose=True, force="--incremental" not in sys.argv)
