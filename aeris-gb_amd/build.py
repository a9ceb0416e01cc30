"""Build libaeris_hip.so (gfx950) in-tree with hipcc.

    python aeris-gb_amd/build.py [--force]

Cross-compiles without a GPU.  The shared library lands next to the sources
(``csrc/libaeris_hip.so``) so that it travels with the tree.
"""
from __future__ import annotations

import importlib.util
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "libaeris_hip.so")
SOURCES = ["api.hip", "gemm.hip", "gemm_persistent.hip", "window_attention.hip", "qkv_window_attention.hip", "window_attention_stream.hip", "norm_modulate.hip", "small_ops.hip", "output_stage.hip", "input_stage.hip"]
HEADERS = ["common.h", "kernels.h", "gemm_common.h", "attention_sweep.h", os.path.join("..", "..", "include", "aeris_hip.h")]
# sources whose transposing LDS reads are inline assembly: their device assembly is checked after every compile
# (asm_check.py says for what); the compile keeps its temporaries for that, in a scratch directory
ASM_CHECKED = {"window_attention.hip", "qkv_window_attention.hip", "window_attention_stream.hip"}
# packed fp32 VALU ops stay off: some of their forms have produced wrong results on this hardware
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _asm_check():
    spec = importlib.util.spec_from_file_location("aeris_asm_check", os.path.join(HERE, "asm_check.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def build(force: bool = False, verbose: bool = True) -> str:
    hipcc = _hipcc()
    hdrs = [os.path.join(CSRC, h) for h in HEADERS]
    objs, jobs = [], []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(CSRC, s.replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, [src] + hdrs):
            jobs.append((s, src, obj))

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed ({r.returncode}):\n{out}")
        if verbose and out.strip():
            print(out, flush=True)

    def compile_one(job):
        name, src, obj = job
        if name not in ASM_CHECKED:
            run([hipcc, *FLAGS, "-c", src, "-o", obj])
            return
        tmp = tempfile.mkdtemp(prefix="aeris_build_")
        try:
            tmp_obj = os.path.join(tmp, os.path.basename(obj))
            run([hipcc, *FLAGS, "-save-temps=obj", "-c", src, "-o", tmp_obj])
            asm = [f for f in os.listdir(tmp) if f.endswith(".s") and "amdgcn" in f]
            if len(asm) != 1:
                raise RuntimeError(f"{name}: expected one device assembly file among the compile's temporaries, found {asm}")
            with open(os.path.join(tmp, asm[0])) as f:
                problems, n_reads = _asm_check().check_text(f.read())
            if n_reads == 0:
                raise RuntimeError(f"{name}: no transposing LDS read in its assembly - is it still one of ASM_CHECKED?")
            if problems:
                raise RuntimeError(f"{name}: the assembly breaks the rules of the inline-assembly LDS reads:\n  " + "\n  ".join(problems[:20]))
            if verbose:
                print(f"{name}: {n_reads} transposing LDS reads checked", flush=True)
            shutil.move(tmp_obj, obj)
        finally:
            shutil.rmtree(tmp, ignore_errors=True)

    with ThreadPoolExecutor(max_workers=min(4, max(1, len(jobs)))) as ex:
        list(ex.map(compile_one, jobs))
    if force or jobs or _stale(LIB, objs):
        run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
