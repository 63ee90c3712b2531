"""Builds and loads the HIP shared objects of `miniinfer_amd/csrc`.

Each source file becomes one shared object with a C interface, built by `hipcc` for gfx950
and loaded with `ctypes`.  A source may be specialised by preprocessor defines (the head
size of the MFMA attention kernels, for one), so what is compiled at a model's first use is
what that model needs.  Built objects live in `csrc/_build/` inside the package (or, when that
is not writable, in a per-user folder under the temp dir); the file name carries a hash of the
sources and flags, so a changed source is rebuilt and an unchanged one is loaded as it is.

There is no fallback: a missing compiler or a failed build raises.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

ARCH = "gfx950"
CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))

# packed 32-bit float instructions are switched off for every kernel of this library
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
               # MFMA results stay in ordinary vector registers: the kernels here read every product's
               # accumulators with vector instructions at once, and copies to and from the accumulation
               # registers were a third of the attention loop's instructions
               "-mllvm", "-amdgpu-mfma-vgpr-form=1"]

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
  pass


def _hipcc() -> str:
  for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
    if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
      return cand
  raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels of "
                   "miniinfer_amd cannot be built, and there is no fallback path")


def _headers() -> List[str]:
  return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _tag(name: str, defines: Sequence[Tuple[str, object]]) -> str:
  h = hashlib.sha256()
  for path in [os.path.join(CSRC, name + ".hip")] + _headers():
    with open(path, "rb") as f:
      h.update(f.read())
  h.update(" ".join(HIPCC_FLAGS).encode())
  h.update(repr(sorted(defines)).encode())
  suffix = "".join(f"-{k}{v}" for k, v in sorted(defines))
  return f"{name}{suffix}-{h.hexdigest()[:10]}"


def build_dirs() -> List[str]:
  """Where built objects are looked for and written, in order of preference."""
  dirs = [os.path.join(CSRC, "_build")]
  env = os.environ.get("MINIINFER_AMD_BUILD_DIR")
  if env:
    dirs.insert(0, env)
  uid = os.getuid() if hasattr(os, "getuid") else 0
  dirs.append(os.path.join(tempfile.gettempdir(), f"miniinfer_amd-build-{uid}"))
  return dirs


def _private_temp_dir(d: str) -> bool:
  """The per-user folder under the temp dir is only used when it belongs to this user and nobody else can write to
  it: a library is loaded from it, and another user of the machine could have made the folder first."""
  uid = os.getuid() if hasattr(os, "getuid") else None
  try:
    os.makedirs(d, mode=0o700, exist_ok=True)
    st = os.lstat(d)
  except OSError:
    return False
  import stat
  if not stat.S_ISDIR(st.st_mode) or (uid is not None and st.st_uid != uid) or (st.st_mode & 0o022):
    return False
  return True


def _usable(d: str) -> bool:
  """Whether built objects may be looked for in `d`: the in-tree folder and an explicitly named one always, the
  shared temp dir's folder only when it is this user's own."""
  return not d.startswith(tempfile.gettempdir() + os.sep) or d == os.environ.get("MINIINFER_AMD_BUILD_DIR") \
      or (os.path.isdir(d) and _private_temp_dir(d))


def _writable_dir() -> str:
  for d in build_dirs():
    try:
      if d.startswith(tempfile.gettempdir() + os.sep) and d != os.environ.get("MINIINFER_AMD_BUILD_DIR"):
        if not _private_temp_dir(d):
          continue
      else:
        os.makedirs(d, exist_ok=True)
      fd, probe = tempfile.mkstemp(prefix=".probe-", dir=d)
      os.close(fd)
      os.unlink(probe)
      return d
    except OSError:
      continue
  raise BuildError(f"no writable folder for built kernels among {build_dirs()} (a folder under the temp dir is "
                   "used only if it belongs to this user and no one else can write to it)")


def find_built(name: str, defines: Sequence[Tuple[str, object]] = ()) -> Optional[str]:
  fn = _tag(name, defines) + ".so"
  for d in build_dirs():
    p = os.path.join(d, fn)
    if os.path.isfile(p) and _usable(d):
      return p
  return None


def compile_module(name: str, defines: Sequence[Tuple[str, object]] = (), force: bool = False,
                   quiet: bool = False) -> str:
  """Build one shared object (unless it is there already and `force` is off); returns its path."""
  if not force:
    p = find_built(name, defines)
    if p:
      return p
  src = os.path.join(CSRC, name + ".hip")
  if not os.path.isfile(src):
    raise BuildError(f"no kernel source {src}")
  out_dir = _writable_dir()
  out = os.path.join(out_dir, _tag(name, defines) + ".so")
  tmp = out + f".tmp{os.getpid()}"
  cmd = [_hipcc()] + HIPCC_FLAGS + ["-I", CSRC] + [f"-D{k}={v}" for k, v in defines] + ["-o", tmp, src]
  what = name + ("" if not defines else " (" + ", ".join(f"{k}={v}" for k, v in defines) + ")")
  if not quiet:
    print(f"[miniinfer_amd] compiling {what} for {ARCH} ...", file=sys.stderr, flush=True)
  t0 = time.time()
  proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          env=dict(os.environ, HOME=os.environ.get("HOME") or tempfile.gettempdir()))
  last = t0
  while True:
    try:
      log, _ = proc.communicate(timeout=5)
      break
    except subprocess.TimeoutExpired:
      if not quiet and time.time() - last >= 15:
        last = time.time()
        print(f"[miniinfer_amd] ... still compiling {what} ({last - t0:.0f} s)", file=sys.stderr, flush=True)
  if proc.returncode != 0:
    try:
      os.unlink(tmp)
    except OSError:
      pass
    raise BuildError(f"hipcc failed for {what} (exit {proc.returncode}):\n{' '.join(cmd)}\n{log}")
  os.replace(tmp, out)
  if not quiet:
    print(f"[miniinfer_amd] compiled {what} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
  return out


def compile_many(jobs: Iterable[Tuple[str, Sequence[Tuple[str, object]]]], force: bool = False,
                 max_workers: int = 8) -> List[str]:
  """Build several objects side by side (hipcc runs in child processes)."""
  from concurrent.futures import ThreadPoolExecutor
  jobs = list(jobs)
  if not jobs:
    return []
  with ThreadPoolExecutor(max_workers=min(max_workers, len(jobs))) as pool:
    return list(pool.map(lambda j: compile_module(j[0], j[1], force=force), jobs))


def load_module(name: str, defines: Sequence[Tuple[str, object]] = ()) -> ctypes.CDLL:
  """The loaded shared object of `csrc/<name>.hip` with these defines; built at first use."""
  defines = tuple(sorted(defines))
  key = name + repr(defines)
  lib = _loaded.get(key)
  if lib is not None:
    return lib
  with _lock:
    lib = _loaded.get(key)
    if lib is None:
      path = compile_module(name, defines)
      lib = ctypes.CDLL(path)
      lib.mi_last_error.restype = ctypes.c_char_p
      _loaded[key] = lib
  return lib


def loaded_objects() -> List[str]:
  return sorted(getattr(lib, "_name", "?") for lib in _loaded.values())
