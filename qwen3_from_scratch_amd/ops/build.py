"""Compile the HIP sources under csrc/ for gfx950 and load them with ctypes.

Each `<module>.hip` becomes `csrc/lib/<module>.so`. A module is built when its
library is missing or was built from other sources or flags (a digest of the
file, the headers it includes and the flags is kept beside it), at the first call of an operation that lives in it; nothing else
is compiled. If the package folder cannot be written, libraries go to a
temporary folder. There is no other implementation to fall back to: a failure
to build or load raises.
"""

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))
ARCH = "gfx950"
FLAGS = [
    "--offload-arch=" + ARCH,
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
MODULES = ("elementwise", "norm", "rotary", "attention", "gemm", "matmul", "sampling", "probes")
# what a module links besides the HIP runtime
LINKS = {"matmul": ["-lhipblaslt"]}

_loaded = {}
_lock = threading.Lock()


class ExtensionError(RuntimeError):
    """The HIP extension could not be built or loaded."""


def _say(message):
    print("[qwen3_from_scratch_amd] " + message, file=sys.stderr, flush=True)


def _hipcc():
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise ExtensionError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _sources(module):
    """The module's .hip file and the headers of this folder that it includes, directly or
    through another header."""
    found, todo = [], [module + ".hip"]
    while todo:
        name = todo.pop()
        if name in found or not os.path.isfile(os.path.join(CSRC, name)):
            continue
        found.append(name)
        with open(os.path.join(CSRC, name), encoding="utf-8", errors="replace") as fh:
            todo += re.findall(r'^\s*#\s*include\s+"([^"]+)"', fh.read(), flags=re.MULTILINE)
    return sorted(found)


def _digest(module):
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + LINKS.get(module, [])).encode())
    for name in _sources(module):
        with open(os.path.join(CSRC, name), "rb") as fh:
            h.update(name.encode())
            h.update(fh.read())
    return h.hexdigest()


def _lib_dirs():
    yield os.path.join(CSRC, "lib")
    yield os.path.join(tempfile.gettempdir(), "qwen3_from_scratch_amd_%d" % os.getuid(), "lib")


def _is_current(lib_dir, module, digest):
    so = os.path.join(lib_dir, module + ".so")
    tag = so + ".digest"
    if not (os.path.isfile(so) and os.path.isfile(tag)):
        return False
    with open(tag) as fh:
        return fh.read().strip() == digest


def compile_module(module, force=False):
    """Compile one module if needed; returns the path of its library."""
    source = os.path.join(CSRC, module + ".hip")
    if not os.path.isfile(source):
        raise ExtensionError("no source %s" % source)
    digest = _digest(module)
    if not force:
        for lib_dir in _lib_dirs():
            if _is_current(lib_dir, module, digest):
                return os.path.join(lib_dir, module + ".so")
    hipcc = _hipcc()
    last_error = None
    for lib_dir in _lib_dirs():
        try:
            os.makedirs(lib_dir, exist_ok=True)
            probe = os.path.join(lib_dir, ".write_probe_%d" % os.getpid())
            with open(probe, "w"):
                pass
            os.remove(probe)
        except OSError as exc:
            last_error = exc
            continue
        so = os.path.join(lib_dir, module + ".so")
        tmp = so + ".tmp%d" % os.getpid()
        cmd = [hipcc] + FLAGS + ["-I", CSRC, source, "-o", tmp]
        if module in LINKS:
            rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))), "lib")
            cmd += ["-L" + rocm_lib] + LINKS[module]
        _say("compiling %s.hip for %s ..." % (module, ARCH))
        started = time.time()
        env = dict(os.environ)
        env.setdefault("HOME", tempfile.gettempdir())
        if not os.path.isdir(env["HOME"]) or not os.access(env["HOME"], os.W_OK):
            env["HOME"] = tempfile.gettempdir()
        proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env)
        done = threading.Event()

        def ticker():
            while not done.wait(15.0):
                _say("  still compiling %s.hip (%d s)" % (module, time.time() - started))

        thread = threading.Thread(target=ticker, daemon=True)
        thread.start()
        out = proc.communicate()[0].decode(errors="replace")
        done.set()
        if proc.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            raise ExtensionError("hipcc failed for %s.hip:\n%s" % (module, out))
        os.replace(tmp, so)
        with open(so + ".digest", "w") as fh:
            fh.write(digest)
        _say("built %s.so in %.1f s" % (module, time.time() - started))
        return so
    raise ExtensionError("no writable folder for the built library: %s" % last_error)


def build_all(force=True):
    """Compile every module (what __graft_entry__.build() calls)."""
    return [compile_module(m, force=force) for m in MODULES]


def library(module):
    """The loaded library of `module`, built first if need be."""
    lib = _loaded.get(module)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(module)
        if lib is None:
            path = compile_module(module)
            try:
                lib = ctypes.CDLL(path)
            except OSError as exc:
                raise ExtensionError("cannot load %s: %s" % (path, exc)) from exc
            _loaded[module] = lib
    return lib


def loaded_libraries():
    return {m: lib._name for m, lib in _loaded.items()}
