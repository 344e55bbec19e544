"""In-tree build of the gfx950 HIP extension.

Invokes hipcc directly (no hipify, no CUDA shims) and links against the
installed PyTorch-ROCm. The kernels are split into GROUPS, one shared
library each (`_kaito_<group>.so`, next to this file so it travels with
the repo snapshot to GPU boxes). A group is compiled and loaded the first
time one of its ops is called, so a model only pays for the kernels it
uses; sources compile to objects in parallel.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import Dict, Iterable, List, Optional

OPS_DIR = Path(__file__).resolve().parent
CSRC = OPS_DIR / "csrc"
OBJ_DIR = OPS_DIR / "_obj"
ARCH = os.environ.get("PYTORCH_ROCM_ARCH", "gfx950")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# group → sources (relative to csrc/). Every group registers its own ops
# with TORCH_LIBRARY_FRAGMENT, so any subset can be loaded.
GROUPS: Dict[str, List[str]] = {
    # norms, activations, rope, paged-cache scatter, top-k
    "core": ["bind_core.cpp", "rmsnorm.hip", "activation.hip", "rope.hip",
             "cache.hip", "topk.hip"],
    # rotary-model attention over the paged cache (decode/prefill/context)
    "attn": ["bind_attn.cpp", "paged_attention.hip",
             "paged_attention_sp.hip", "prefill_attention.hip",
             "context_attention.hip", "diag.hip", "mfma_probe.hip"],
    "mla": ["bind_mla.cpp", "mla_attention.hip"],
    "moe": ["bind_moe.cpp", "moe.hip"],
    "quant": ["bind_quant.cpp", "w4a16.hip", "lora.hip"],
    "comm": ["bind_comm.cpp", "allreduce_rmsnorm.hip"],
    # hybrid stacks (each source registers its own ops). "mix": what every
    # hybrid design uses — short convolutions, window attention over the
    # paged cache, f32 residual norms, element-wise gates
    "mix": ["causal_conv.hip", "window_attention.hip", "residual_norm.hip",
            "gated_act.hip"],
    # gated delta rule and real-gated linear recurrence
    "delta": ["delta_rule.hip", "rglru.hip"],
    # scalar-decay matrix recurrences: mLSTM, state-space duality
    "decay": ["decay_recurrence.hip"],
    # latent attention over a paged low-rank cache, hashed bigram embedding
    "latent": ["latent_attention.hip"],
    # matrix recurrences with a decay per state row: generalized delta
    # rule, gated linear attention with a tied write gate
    "diag": ["diag_delta.hip"],
}


def so_path(group: str) -> Path:
    return OPS_DIR / f"_kaito_{group}.so"


# kept for callers that print where the extension lives
SO_PATH = so_path("core")


def _torch_paths():
    import torch
    from torch.utils import cpp_extension as ce

    return ce.include_paths(), ce.library_paths(), torch.compiled_with_cxx11_abi()


def _sources(group: str) -> List[Path]:
    return [CSRC / s for s in GROUPS[group]]


def _headers() -> List[Path]:
    return sorted(CSRC.glob("*.h"))


def needs_build(group: str) -> bool:
    so = so_path(group)
    if not so.exists():
        return True
    t = so.stat().st_mtime
    return any(s.stat().st_mtime > t for s in _sources(group) + _headers())


def _compile_cmd(src: Path, obj: Path, includes, cxx11) -> List[str]:
    cmd = [
        HIPCC, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-c",
        "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__=1",
        f"-D_GLIBCXX_USE_CXX11_ABI={1 if cxx11 else 0}",
        "-fno-gpu-rdc", "-Wno-unused-result", "-Wno-unknown-attributes",
        # packed-f32 VALU forms are kept out of every kernel
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    ]
    for inc in includes:
        cmd += ["-I", inc]
    cmd += [str(src), "-o", str(obj)]
    return cmd


def build(verbose: bool = True, force: bool = False,
          groups: Optional[Iterable[str]] = None) -> List[Path]:
    """Compile and link the given groups (default: all). With force=False
    a group whose library is newer than its sources is left alone."""
    todo = [g for g in (list(groups) if groups is not None else list(GROUPS))
            if force or needs_build(g)]
    if not todo:
        return [so_path(g) for g in (groups or GROUPS)]
    includes, libdirs, cxx11 = _torch_paths()
    OBJ_DIR.mkdir(exist_ok=True)
    jobs = []
    for g in todo:
        for src in _sources(g):
            obj = OBJ_DIR / (src.name + ".o")
            jobs.append((src, obj))
    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "0"))
                         or (os.cpu_count() or 4), 16))

    def run(job):
        src, obj = job
        cmd = _compile_cmd(src, obj, includes, cxx11)
        if verbose:
            print("[kaito_amd] hipcc", src.name, file=sys.stderr, flush=True)
        subprocess.run(cmd, check=True, stderr=None if verbose
                       else subprocess.PIPE)

    with ThreadPoolExecutor(workers) as ex:
        list(ex.map(run, jobs))
    out = []
    for g in todo:
        so = so_path(g)
        tmp = so.with_suffix(f".so.tmp{os.getpid()}")
        cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC",
               "-fno-gpu-rdc"]
        cmd += [str(OBJ_DIR / (s.name + ".o")) for s in _sources(g)]
        for ld in libdirs:
            cmd += ["-L", ld, f"-Wl,-rpath,{ld}"]
        cmd += ["-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip",
                "-L/opt/rocm/lib", "-lamdhip64", "-o", str(tmp)]
        subprocess.run(cmd, check=True)
        os.replace(tmp, so)          # atomic: a reader never sees half a file
        out.append(so)
        if verbose:
            print("[kaito_amd] linked", so.name, file=sys.stderr, flush=True)
    return out


if __name__ == "__main__":
    args = [a for a in sys.argv[1:] if not a.startswith("--")]
    build(force="--force" in sys.argv, groups=args or None)
