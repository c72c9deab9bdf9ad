"""Build and load ``libpagedserve_hip.so``, the engine's gfx950 kernels.

The library is plain HIP behind a C interface (``csrc/pagedserve_hip.h``), compiled
with ``hipcc --offload-arch=gfx950`` and called through ``ctypes`` with device
pointers of torch tensors and the current HIP stream.  It is built inside the
package (``pagedserve_amd/_lib``) when that folder can be written, else in a
per-user folder under the temporary directory; a hash of the sources next to the
library tells whether it is current.  Nothing here falls back to another
implementation: if the library cannot be built or loaded, the error is raised.
"""

import ctypes
import hashlib
import os
import shutil
import stat
import subprocess
import sys
import tempfile
import time

import torch  # noqa: F401  (loads the HIP runtime that the library links against)

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE_DIR = os.path.join(PACKAGE_DIR, "csrc")
LIB_NAME = "libpagedserve_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops is switched off: some packed float forms have given wrong results on
# this hardware generation without any error.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# Per source: matrix products that accumulate in ordinary vector registers.  Kernels that go on
# computing with the results (softmax, wide epilogues) then need no copies from the
# accumulation registers; the skinny decode products are better off without.
EXTRA_FLAGS = {
    "attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "attention_mixed.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "gemm_tiled_bf16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


class KernelLibraryError(RuntimeError):
    pass


def _sources():
    names = sorted(name for name in os.listdir(SOURCE_DIR) if name.endswith(".hip"))
    headers = sorted(name for name in os.listdir(SOURCE_DIR) if name.endswith(".h"))
    return names, headers


def source_hash() -> str:
    digest = hashlib.sha256()
    names, headers = _sources()
    for name in names + headers:
        digest.update(name.encode())
        with open(os.path.join(SOURCE_DIR, name), "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    digest.update(repr(sorted(EXTRA_FLAGS.items())).encode())
    return digest.hexdigest()[:16]


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise KernelLibraryError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def in_tree_dir() -> str:
    return os.path.join(PACKAGE_DIR, "_lib")


def _writable(folder) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe-{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


_PRIVATE_DIR = None


def _fallback_dir() -> str:
    """Where the library is built and looked for when the tree cannot be written: a folder
    under the temporary directory that belongs to this user alone.  The name can be guessed, so
    a folder of that name that someone else made, or that others may write, is never used (a
    library planted there would be loaded): a fresh private folder takes its place for this
    process."""
    global _PRIVATE_DIR
    if _PRIVATE_DIR is not None:
        return _PRIVATE_DIR
    path = os.path.join(tempfile.gettempdir(), f"pagedserve_amd-{os.getuid()}")
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        status = os.lstat(path)
        mine = (stat.S_ISDIR(status.st_mode) and status.st_uid == os.getuid()
                and not status.st_mode & 0o022)
    except OSError:
        mine = False
    _PRIVATE_DIR = path if mine else tempfile.mkdtemp(prefix="pagedserve_amd-")
    return _PRIVATE_DIR


def _say(message, verbose):
    if verbose:
        print(f"[pagedserve_amd] {message}", file=sys.stderr, flush=True)


def build(target_dir=None, verbose=True, jobs=None) -> str:
    """Compile every ``csrc/*.hip`` for gfx950 and link the shared library.

    Always compiles; returns the path of the library."""
    hipcc = _hipcc()
    if target_dir is None:
        target_dir = in_tree_dir() if _writable(in_tree_dir()) else _fallback_dir()
    os.makedirs(target_dir, exist_ok=True)
    object_dir = os.path.join(target_dir, "_build")
    os.makedirs(object_dir, exist_ok=True)
    names, _ = _sources()
    jobs = jobs or min(len(names), max(1, min(16, os.cpu_count() or 1)))
    _say(f"compiling {len(names)} HIP sources for {ARCH} with {hipcc} ({jobs} at a time)", verbose)
    started = time.time()
    pending = list(names)
    running = {}
    objects = []
    failed = []
    last_note = time.time()
    while pending or running:
        while pending and len(running) < jobs:
            name = pending.pop(0)
            obj = os.path.join(object_dir, name[:-4] + ".o")
            objects.append(obj)
            command = [hipcc] + HIPCC_FLAGS + EXTRA_FLAGS.get(name, []) + ["-I", SOURCE_DIR, "-c",
                                              os.path.join(SOURCE_DIR, name), "-o", obj]
            running[name] = subprocess.Popen(command, stdout=subprocess.PIPE,
                                             stderr=subprocess.STDOUT, text=True)
        for name, process in list(running.items()):
            if process.poll() is None:
                continue
            output = process.stdout.read()
            del running[name]
            if process.returncode != 0:
                failed.append((name, output))
            else:
                _say(f"  compiled {name} ({time.time() - started:.0f} s)", verbose)
        if running:
            time.sleep(0.1)
            if time.time() - last_note > 10:
                _say(f"  still compiling: {', '.join(sorted(running))}", verbose)
                last_note = time.time()
    if failed:
        text = "\n".join(f"--- {name} ---\n{output}" for name, output in failed)
        raise KernelLibraryError(f"hipcc failed:\n{text}")
    library = os.path.join(target_dir, LIB_NAME)
    temporary = library + f".tmp-{os.getpid()}"
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", temporary] + objects
    result = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if result.returncode != 0:
        raise KernelLibraryError(f"linking {LIB_NAME} failed:\n{result.stdout}")
    os.replace(temporary, library)
    with open(os.path.join(target_dir, LIB_NAME + ".hash"), "w") as handle:
        handle.write(source_hash())
    _say(f"built {library} in {time.time() - started:.0f} s", verbose)
    return library


def _current(folder) -> bool:
    library = os.path.join(folder, LIB_NAME)
    stamp = library + ".hash"
    if not (os.path.isfile(library) and os.path.isfile(stamp)):
        return False
    with open(stamp) as handle:
        return handle.read().strip() == source_hash()


def find_or_build(verbose=True) -> str:
    """The path of a library that matches the sources, building it if there is none."""
    for folder in (in_tree_dir(), _fallback_dir()):
        if _current(folder):
            return os.path.join(folder, LIB_NAME)
    return build(verbose=verbose)


_LIBRARY = None


def load_library() -> ctypes.CDLL:
    """The loaded kernel library (built on first use when it is missing or stale)."""
    global _LIBRARY
    if _LIBRARY is None:
        path = find_or_build()
        try:
            _LIBRARY = ctypes.CDLL(path)
        except OSError as error:
            raise KernelLibraryError(f"cannot load {path}: {error}") from error
        _LIBRARY.ps_last_error.restype = ctypes.c_char_p
        _LIBRARY.path = path
    return _LIBRARY
