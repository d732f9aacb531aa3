"""Compiling the HIP sources and finding what is compiled.

Each source under `csrc/` becomes one shared library named after the hash of
its text (and of the shared header and the flags), so a library never outlives
the source it was built from. A library is compiled when it is first needed and
kept beside the sources; if that folder cannot be written, under the user's
cache folder or the temporary folder. While hipcc runs a line is printed every
few seconds.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
MODULES = ("elementwise", "gemm", "attention", "sampling", "probe")
ARCH = "gfx950"
FLAGS = ["-O3", f"--offload-arch={ARCH}", "-shared", "-fPIC", "-std=c++17",
         # packed float32 instructions are kept out of the generated code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

_locks = {m: threading.Lock() for m in MODULES}
_SOURCES: Dict[str, str] = {m: os.path.join(CSRC, f"{m}.hip") for m in MODULES}


def register_module(name: str, source: str) -> None:
    """A kernel module from outside the package: a part that needs a kernel of its own names its source
    here (and its C signatures with `hip.register_signatures`), and reaches it through `HipOps.call`. The
    library is built like the others, beside its source (folder `lib/`), and `common.h` is on its include path."""
    if name in _SOURCES and os.path.abspath(_SOURCES[name]) != os.path.abspath(source):
        raise BuildError(f"a kernel module named {name!r} is registered already, from {_SOURCES[name]}")
    _SOURCES[name] = source
    _locks.setdefault(name, threading.Lock())


def modules() -> List[str]:
    return list(_SOURCES)


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[transformers_neuronx_amd] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


def source_hash(module: str) -> str:
    h = hashlib.sha256()
    src = _SOURCES[module]
    own_header = os.path.join(os.path.dirname(src), f"tnx_{module}.h")   # its entry points: not every module has one
    for path in (src, os.path.join(CSRC, "common.h"), own_header):
        if path == own_header and not os.path.exists(path):
            continue
        with open(path, "rb") as fp:
            h.update(fp.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _lib_dirs(module: Optional[str] = None) -> List[str]:
    src_dir = os.path.dirname(_SOURCES[module]) if module in _SOURCES else CSRC
    dirs = [os.path.join(src_dir, "lib")]
    home = os.environ.get("XDG_CACHE_HOME") or (os.path.join(os.environ["HOME"], ".cache")
                                                if os.environ.get("HOME") else None)
    if home:
        dirs.append(os.path.join(home, "transformers_neuronx_amd"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"transformers_neuronx_amd-{os.getuid()}"))
    return dirs


def lib_name(module: str) -> str:
    return f"tnx_{module}-{source_hash(module)}.so"


def find_library(module: str) -> Optional[str]:
    name = lib_name(module)
    for d in _lib_dirs(module):
        path = os.path.join(d, name)
        if os.path.exists(path):
            return path
    return None


def _writable_dir(module: Optional[str] = None) -> str:
    for d in _lib_dirs(module):
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}-{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no folder to keep compiled kernels in: tried " + ", ".join(_lib_dirs(module)))


def compile_module(module: str, force: bool = False) -> str:
    """Compile `csrc/<module>.hip` for gfx950; returns the library's path."""
    if module not in _SOURCES:
        raise BuildError(f"unknown kernel module {module!r}")
    with _locks[module]:
        if not force:
            found = find_library(module)
            if found:
                return found
        hipcc = find_hipcc()
        if hipcc is None:
            raise BuildError(f"the HIP kernels of '{module}' are not built and hipcc was not found "
                             "(looked at $HIPCC, PATH and /opt/rocm/bin)")
        out_dir = _writable_dir(module)
        out = os.path.join(out_dir, lib_name(module))
        tmp = f"{out}.{os.getpid()}.tmp"
        cmd = [hipcc] + FLAGS + ["-I", CSRC, _SOURCES[module], "-o", tmp]
        _log(f"compiling {module}.hip for {ARCH} ...")
        start = time.time()
        proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=out_dir)
        lines: List[str] = []
        reader = threading.Thread(target=lambda: lines.extend(proc.stdout.readlines()), daemon=True)
        reader.start()
        while True:
            try:
                proc.wait(timeout=10)
                break
            except subprocess.TimeoutExpired:
                _log(f"still compiling {module}.hip ({int(time.time() - start)} s)")
        reader.join()
        text = "".join(l for l in lines if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            raise BuildError(f"hipcc failed on {module}.hip:\n{text}")
        os.replace(tmp, out)
        for old in os.listdir(out_dir):   # libraries of earlier versions of this source
            if old.startswith(f"tnx_{module}-") and old.endswith(".so") and old != os.path.basename(out):
                try:
                    os.remove(os.path.join(out_dir, old))
                except OSError:
                    pass
        _log(f"compiled {module}.hip in {time.time() - start:.1f} s -> {out}")
        return out


def build_all(force: bool = True) -> Dict[str, str]:
    """Compile every module, side by side (the "does it build" check)."""
    out: Dict[str, str] = {}
    errors: List[str] = []

    def work(m):
        try:
            out[m] = compile_module(m, force)
        except BuildError as e:   # collected and raised together
            errors.append(str(e))

    threads = [threading.Thread(target=work, args=(m,)) for m in modules()]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise BuildError("\n".join(errors))
    return out
