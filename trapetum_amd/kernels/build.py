"""Compiling the HIP sources for gfx950 into shared libraries next to them.

One core library (norms, embedding, RoPE + cache write, matrix products, plain attention, sampling) and one
attention library per head size, compiled when a model first needs it.  Objects and libraries go to
csrc/_build inside the package, or to a per-user folder under the temporary directory if the package folder
cannot be written.  A stamp (hash of sources and flags) tells whether a library still matches its sources.
"""
import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]
CORE_SOURCES = ["elementwise.hip", "gemm.hip", "gemm_skinny.hip", "gemm_mfma.hip", "gemv.hip", "gemm_rows8.hip", "attention_simple.hip", "sampling.hip", "probes.hip"]
ATTN_SOURCES = ["attention_mfma.hip", "attention_prefill.hip"]      # decode steps; steps of many queries
_NOISE = "is not a recognized feature for this target"


class BuildError(RuntimeError):
    pass


def _say(msg):
    print(f"[trapetum_amd] {msg}", file=sys.stderr, flush=True)


def build_dir():
    d = os.path.join(CSRC, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"trapetum_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _headers(sources):
    """The headers of csrc/ that the sources include, directly or through one another."""
    seen, todo = set(), list(sources)
    while todo:
        with open(os.path.join(CSRC, todo.pop()), "r", errors="replace") as f:
            for line in f:
                line = line.strip()
                if line.startswith("#include \""):
                    name = line.split('"')[1]
                    if name not in seen and os.path.isfile(os.path.join(CSRC, name)):
                        seen.add(name)
                        todo.append(name)
    return sorted(seen)


def _stamp(sources, defines):
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + list(defines)).encode())
    for name in list(sources) + _headers(sources):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    return h.hexdigest()


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise BuildError("hipcc was not found: the HIP kernels cannot be compiled on this machine")
    return exe


def _run(cmd, what):
    p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    t0 = time.time()
    last = t0
    while True:
        try:
            out, _ = p.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if time.time() - last >= 20:
                _say(f"still compiling {what} ({int(time.time() - t0)} s)")
                last = time.time()
    out = "\n".join(l for l in (out or "").splitlines() if _NOISE not in l)
    if p.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{out}")
    return out


def library_path(name):
    return os.path.join(build_dir(), f"lib{name}.so")


def is_current(name, sources, defines):
    lib = library_path(name)
    stamp = lib + ".stamp"
    if not (os.path.isfile(lib) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == _stamp(sources, defines)


def build_library(name, sources, defines=(), force=False):
    """Compile `sources` (in csrc/) into lib<name>.so; returns its path."""
    defines = list(defines)
    lib = library_path(name)
    if not force and is_current(name, sources, defines):
        return lib
    cc = hipcc()
    d = build_dir()
    _say(f"compiling {name} for {ARCH} ({len(sources)} files) into {d}")
    objs = []

    def one(src):
        obj = os.path.join(d, f"{name}.{os.path.splitext(src)[0]}.{os.getpid()}.o")
        _run([cc] + FLAGS + defines + ["-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj], src)
        return obj
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        objs = list(ex.map(one, sources))
    tmp = f"{lib}.{os.getpid()}.tmp"
    _run([cc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs, f"lib{name}.so")
    os.replace(tmp, lib)                      # atomic: another process never sees half a library
    for o in objs:
        os.remove(o)
    with open(lib + ".stamp", "w") as f:
        f.write(_stamp(sources, defines))
    _say(f"built {lib}")
    return lib


def build_core(force=False):
    return build_library("trapetum_core", CORE_SOURCES, force=force)


def attn_name(head_dim):
    return f"trapetum_attn_hd{head_dim}"


def build_attention(head_dim, force=False):
    return build_library(attn_name(head_dim), ATTN_SOURCES, [f"-DTP_HD={head_dim}"], force=force)
