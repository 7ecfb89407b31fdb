"""Builds fast_ops_amd/libfastops_hip.so from fast_ops_amd/csrc/*.hip with hipcc for gfx950.

Replaces the reference's import-time JIT builds (fast_ops/flash_attention/flash_attention.py:13-25,
fast_ops/lion/lion_optimizer.py:15-26) and its setup.py (setup.py:4-18) with one ahead-of-time shared library that
has a C ABI and no torch or pybind11 dependency. hipcc cross-compiles without a GPU.

Run ``python -m fast_ops_amd.build`` (add ``--force`` to rebuild everything). ``--ablations`` additionally compiles the
timing ablations of the attention forward (kernel variants that leave work out and produce wrong results by design, for
measuring what each part of the kernel costs); a default build contains none of them and ``fo_tune_set`` refuses
their variant numbers.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "obj")
LIB_PATH = os.path.join(HERE, "libfastops_hip.so")

ARCH = "gfx950"
COMMON_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",   # the direct-to-LDS copies name m0, a reserved register, as a clobber
    # packed fp32 instructions stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# per-source extra flags. lion.hip must not contract a*b+c on its own: its rounding points are part of its contract.
SOURCES = {
    "capi.hip": [],
    "lion.hip": ["-ffp-contract=off"],
    "lion_typed.hip": ["-ffp-contract=off"],
    # attn_fwd.hip and attn_bwd.hip lay their inner loops out as fully unrolled micro-groups; the default size limit for
    # "#pragma unroll" would silently leave them rolled, with their register arrays in scratch memory.
    # (attn_fwd.hip and attn_bwd.hip themselves are the C ABI and the kernel choice; their kernels are compiled as four
    # units each, one per operand type and head_dim, which include them - in parallel, they are what takes the
    # compiler's time)
    "attn_fwd.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_fwd_bf16_d64.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_fwd_bf16_d128.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_fwd_f16_d64.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_fwd_f16_d128.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_bwd.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_bwd_bf16_d64.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_bwd_bf16_d128.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_bwd_f16_d64.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "attn_bwd_f16_d128.hip": ["-mllvm", "-pragma-unroll-threshold=400000"],
    "dropout_mask.hip": [],
}
# sources that other sources include (a change in one of them makes every object stale, like a header's)
INCLUDED_SOURCES = ["attn_fwd.hip", "attn_bwd.hip"]
# sources whose generated assembly is checked by asm_lint: source -> regular expression of the kernel symbols to check
# (the instantiations with a non-zero last template argument are timing experiments with wrong results by design)
# (attn_fwd_wide_kernel<T, D, CAUSAL, QB, DBG, BM>: DBG is the last but one)
_PIPE = r"attn_bwd_dkdv_pipe_kernel"
_WIDE = r"attn_fwd_wide_kernel.*ELi0ELi\d+ELb[01]EEEvNS_10AttnParamsE"
ASM_LINTED = {"attn_fwd_bf16_d64.hip": _WIDE, "attn_fwd_bf16_d128.hip": _WIDE, "attn_fwd_f16_d64.hip": _WIDE, "attn_fwd_f16_d128.hip": _WIDE,
              "attn_bwd_bf16_d64.hip": _PIPE, "attn_bwd_bf16_d128.hip": _PIPE, "attn_bwd_f16_d64.hip": _PIPE, "attn_bwd_f16_d128.hip": _PIPE}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the ROCm toolchain is required to build libfastops_hip.so")
    return exe


def _newest_header_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))] + [os.path.join(CSRC, f) for f in INCLUDED_SOURCES]
    paths.append(os.path.join(os.path.dirname(HERE), "include", "fastops.h"))
    return max(os.path.getmtime(p) for p in paths if os.path.exists(p))


def _run_hipcc(cmd: list, src: str, verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only target feature and says so; everything else is shown
    err = "\n".join(l for l in res.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)


def _compile_one(hipcc: str, src: str, extra: list, force: bool, verbose: bool) -> str:
    stem = os.path.splitext(src)[0]
    obj = os.path.join(OBJ_DIR, stem + ".o")
    extra = extra + _EXTRA_DEFINES
    src_path = os.path.join(CSRC, src)
    stale = force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src_path), _newest_header_mtime())
    if not stale:
        return obj
    if src not in ASM_LINTED:
        _run_hipcc([hipcc] + COMMON_FLAGS + extra + ["-c", src_path, "-o", obj], src, verbose)
        return obj
    # Kernels with inline-assembly MFMAs: first without wait states in front of the MFMAs of the inner loops, keeping
    # the device assembly, which is then checked for the hazards the compiler cannot see inside an asm statement. If the
    # check finds one, compile again with the wait states.
    from .asm_lint import lint_file, lint_m0_file

    def compile_and_lint(nops: int):
        _run_hipcc([hipcc] + COMMON_FLAGS + extra + [f"-DFO_MFMA_NOPS={nops}", "-save-temps=obj", "-c", src_path, "-o", obj], src, verbose)
        asm = os.path.join(OBJ_DIR, f"{stem}-hip-amdgcn-amd-amdhsa-{ARCH}.s")
        if not os.path.exists(asm):
            raise RuntimeError(f"{src}: {asm} was not produced, the generated assembly cannot be checked")
        problems = lint_file(asm, ASM_LINTED[src])
        # the direct-to-LDS copies are inline assembly too: M0 written and read back to back has no fallback build, it is
        # an error in the source
        m0_problems = lint_m0_file(asm)
        for f in os.listdir(OBJ_DIR):           # the other intermediate files are large and of no further use
            if f.startswith(stem + "-") or f.startswith(stem + ".hip-"):
                os.remove(os.path.join(OBJ_DIR, f))
        if m0_problems:
            raise RuntimeError(f"{src}: {len(m0_problems)} LDS-DMA instruction(s) issued directly after a write of M0, e.g. {m0_problems[0]}")
        if any("no function matches" in p for p in problems):
            raise RuntimeError(f"{src}: the assembly check found no kernel to look at ({ASM_LINTED[src]!r} is out of date)")
        return problems

    problems = compile_and_lint(0)
    if problems:
        if verbose:
            print(f"{src}: {len(problems)} MFMA hazard(s) without wait states, e.g. {problems[0]}\n  -> compiling with wait states", flush=True)
        # the object that is linked is the one that was checked: the build with wait states goes through the same check
        # (a hazard that remains there is an error in the source)
        problems = compile_and_lint(1)
        if problems:
            raise RuntimeError(f"{src}: {len(problems)} MFMA hazard(s) remain with wait states in front of every MFMA, e.g. {problems[0]}")
    elif verbose:
        print(f"{src}: inline-assembly MFMAs checked, no hazard", flush=True)
    return obj


_EXTRA_DEFINES: list = []


def build_library(force: bool = False, verbose: bool = True, ablations: bool = False) -> str:
    """Compiles every HIP source for gfx950 and links the shared library. Returns the library path."""
    global _EXTRA_DEFINES
    _EXTRA_DEFINES = ["-DFO_ABLATIONS=1"] if ablations else []
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    # objects compiled with other defines than this build's (an ablation build before a default one) are stale
    stamp = os.path.join(OBJ_DIR, "defines.txt")
    want = " ".join(_EXTRA_DEFINES)
    if not os.path.exists(stamp) or open(stamp).read() != want:
        force = True
        with open(stamp, "w") as f:
            f.write(want)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda kv: _compile_one(hipcc, kv[0], kv[1], force, verbose), SOURCES.items()))
    need_link = force or not os.path.exists(LIB_PATH) or any(os.path.getmtime(o) > os.path.getmtime(LIB_PATH) for o in objs)
    if need_link:
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv or "--ablations" in sys.argv, ablations="--ablations" in sys.argv))
