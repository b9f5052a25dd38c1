"""Build libllmk_gfx950.so from csrc/*.hip with hipcc (cross-compiles without a GPU).

    python -m llm_kernels_amd.build [-j N]

The library lands next to this file so that it travels with the source tree.
"""
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libllmk_gfx950.so")

# -packed-fp32-ops off: hipcc must not form v_pk_{add,mul,fma}_f32 from scalar float code
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    cmd = [hipcc(), *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def _assembly(src):
    """Device assembly of one source (same flags as the object), for the static check of check_asm.py."""
    out = os.path.join(OBJ, os.path.basename(src)[:-4] + ".s")
    cmd = [hipcc(), *FLAGS, "-S", "--cuda-device-only", src, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return out


# what tells that a source hand-issues loads into registers: the loaders themselves, the header of the ring
# kernels, or a tile-kernel kind whose weight rows are expanded from hand-loaded packed words
_ASM_LOAD_MARKS = ('asm volatile("global_load_dword', "ring_load_", "asm_load_", "stream_ring.hpp",
                   "K_W4NK", "K_W4MARLIN", "K_W4A8")


def _has_asm_register_loads(src):
    """True when this source itself names hand-issued register loads (directly, by including the ring header, or
    by instantiating a tile-kernel kind that uses them): its assembly must then show at least one."""
    text = open(src).read()
    return any(m in text for m in _ASM_LOAD_MARKS)


def build(jobs=None, verbose=True):
    from . import check_asm
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
    jobs = jobs or min(8, len(srcs))
    # Kernels that load registers from inline asm are only correct while the compiler never touches the
    # destination before the hand-placed wait: prove it on the assembly of this very build, or fail.  EVERY
    # source is checked (a source without such loads has nothing to flag); a source whose text, or a header it
    # includes, contains hand-issued loads must show at least one in its assembly, otherwise the check has gone blind.
    with cf.ThreadPoolExecutor(jobs) as ex:
        asm_jobs = [(s, ex.submit(_assembly, s)) for s in srcs]
        objs = list(ex.map(_compile, srcs))
        checked = 0
        for src, j in asm_jobs:
            n, problems = check_asm.check_file(j.result())
            checked += n
            if problems:
                raise RuntimeError("hand-issued register loads are not safe in this build:\n  " + "\n  ".join(problems[:20]))
            if n == 0 and _has_asm_register_loads(src):
                raise RuntimeError("check_asm found no hand-issued loads in %s although its text has them: the check "
                                   "no longer sees them" % src)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LIB, "from", len(srcs), "sources;", checked, "hand-issued register loads verified in the assembly")
    return LIB


if __name__ == "__main__":
    j = None
    if "-j" in sys.argv:
        j = int(sys.argv[sys.argv.index("-j") + 1])
    build(j)
