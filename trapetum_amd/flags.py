"""Run-time switches, read once from the environment (the reference reads its TRAPETUM_* variables once into
statics the same way: runtime/src/lib.rs:1400-1403, runtime/cuda/codebook_gemv.cu:32-36).

TRAPETUM_AMD_DEBUG_DUMP=1   one stderr line per layer and stage of every step, in the reference's format
                            `[ldump] L= stage= l2= absmax= mean=` (runtime/src/lib.rs:1384-1389), and the five largest
                            logits of the step's last wanted row (`[ldump] top5=`, :1392-1397); to find the first layer
                            and stage where two runs part.
TRAPETUM_AMD_PROFILE=1      the time of every kernel-library call by HIP events, summed per entry point and printed
                            to stderr when the process ends (the reference times its ops one by one behind a switch
                            too: runtime/src/lib.rs:3218-3245).
TRAPETUM_AMD_FORCE_PLAIN=1  bfloat16 products and attention on the plain kernels instead of the matrix-core ones: the
                            same formulas with one fixed order of additions, to tell a kernel's fault from a model's.
Each of the first two makes every step wait for the device and switches HIP graphs off.
"""
import functools
import os


@functools.lru_cache(maxsize=None)
def _on(name):
    return os.environ.get(name, "") == "1"


def debug_dump():
    return _on("TRAPETUM_AMD_DEBUG_DUMP")


def profile():
    return _on("TRAPETUM_AMD_PROFILE")


def force_plain():
    return _on("TRAPETUM_AMD_FORCE_PLAIN")


def graphs_allowed():
    return not (debug_dump() or profile())
