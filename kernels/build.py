"""In-tree build of the CDNA4 HIP extensions.

Direct hipcc invocation (no hipify, no CUDA-compat layer): compiles the
kernel sources plus their torch bindings for gfx950 and links the shared
objects under vllm_tgis_adapter_amd/.  The built .so files travel with the
repo snapshot to GPU boxes (a JIT cache would not).

Several extensions, so that a model only builds the ones it uses
(``vllm_tgis_adapter_amd.models.native_extensions`` names them per model):

``_C``      the llama/mixtral/opt kernel set (every kernels/*.hip that is not
            listed for another extension) + bindings.cpp, bindings_attn.cpp
``_C_attn`` only the paged grouped-query attention kernels of ``_C`` (generic
            and MFMA) + bindings_attn.cpp, module_attn.cpp
``_C_seq``  f32-residual-stream ops (RMS and layer norms), short causal
            convolution with per-sequence state, grouped-query attention of
            any shape, recurrences with per-sequence state, two-norm blocks,
            rotation + cache write, gates, expert routing, the grouped expert
            product, token shift, chunk-masked differential attention pieces
            + bindings_seq.cpp, bindings_rec.cpp, bindings_par.cpp,
            bindings_mix.cpp
``_C_lat``  windowed latent attention with sinks + bindings_lat.cpp
"""

from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

REPO = Path(__file__).resolve().parent.parent
KERNELS = REPO / "kernels"
PKG = REPO / "vllm_tgis_adapter_amd"
ARCH = os.environ.get("PYTORCH_ROCM_ARCH", "gfx950")

_SEQ_SOURCES = ["stream_ops.hip", "canon_conv.hip", "layer_norm_stream.hip",
                "paged_attention_any.hip", "recurrent_scan.hip", "gated_block.hip",
                "mix_ops.hip"]
# kernels without torch types that more than one extension links
_SHARED_SOURCES = ["moe_gemm.hip"]
_LAT_SOURCES = ["latent_attention.hip", "latent_attention_mfma.hip"]
_ATTN_SOURCES = ["attention.hip", "attention_decode_mfma.hip",
                 "attention_prefill_mfma.hip", "attention_prefill_mfma_v2.hip"]

EXTENSIONS = {
    "_C": dict(
        sources=lambda: [p for p in sorted(KERNELS.glob("*.hip"))
                         if p.name not in _SEQ_SOURCES + _LAT_SOURCES]
        + [KERNELS / "bindings.cpp", KERNELS / "bindings_attn.cpp"],
    ),
    "_C_attn": dict(
        sources=lambda: [KERNELS / n for n in _ATTN_SOURCES]
        + [KERNELS / "bindings_attn.cpp", KERNELS / "module_attn.cpp"],
    ),
    "_C_seq": dict(
        sources=lambda: [KERNELS / n for n in _SEQ_SOURCES + _SHARED_SOURCES]
        + [KERNELS / "bindings_seq.cpp", KERNELS / "bindings_rec.cpp",
           KERNELS / "bindings_par.cpp", KERNELS / "bindings_mix.cpp"],
    ),
    "_C_lat": dict(
        sources=lambda: [KERNELS / n for n in _LAT_SOURCES] + [KERNELS / "bindings_lat.cpp"],
    ),
}
OUT = PKG / "_C.so"


def ext_path(name: str) -> Path:
    return PKG / f"{name}.so"


def build_ext(name: str, verbose: bool = True, force: bool = False) -> Path:
    import torch
    import torch.utils.cpp_extension as ce

    sources = EXTENSIONS[name]["sources"]()
    out = ext_path(name)
    common_h = KERNELS / "common.h"
    if out.exists() and not force:
        newest_src = max(p.stat().st_mtime for p in sources + [common_h])
        if out.stat().st_mtime > newest_src:
            if verbose:
                print(f"[kernels/build] {out} up to date")
            return out

    include_dirs = ce.include_paths() + [sysconfig.get_path("include")]
    torch_lib = Path(torch.__file__).parent / "lib"
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)

    build_dir = KERNELS / "build"
    build_dir.mkdir(exist_ok=True)

    common_flags = [
        f"--offload-arch={ARCH}",
        "-O3",
        "-std=c++17",
        "-fPIC",
        # packed-f32 VALU forms are kept out of the generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        f"-DTORCH_EXTENSION_NAME={name}",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-D__HIP_PLATFORM_AMD__=1",
        "-DUSE_ROCM=1",
        "-DHIPBLAS_V2",
        "-fno-gpu-rdc",
        "-Wno-unused-result",
        "-Wno-switch-bool",
        "-Wno-unknown-warning-option",
    ] + [f"-I{d}" for d in include_dirs]

    objects = []
    jobs = []
    # sources holding a PYBIND11_MODULE bake the extension's name in; all
    # others are shared between extensions as they are
    module_sources = {"bindings.cpp", "bindings_seq.cpp", "bindings_lat.cpp", "module_attn.cpp"}
    for src in sources:
        obj = build_dir / (src.stem + ".o")
        assert src.name in module_sources or "TORCH_EXTENSION_NAME" not in src.read_text()
        objects.append(obj)
        if obj.exists() and not force and obj.stat().st_mtime > max(
            src.stat().st_mtime, common_h.stat().st_mtime
        ):
            continue
        jobs.append(["hipcc", "-c", str(src), "-o", str(obj)] + common_flags)

    def _run(cmd):
        if verbose:
            print("[kernels/build]", " ".join(cmd[:4]), "...", flush=True)
        subprocess.run(cmd, check=True)

    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "0"))
                         or min(8, os.cpu_count() or 1)))
    if jobs:
        with ThreadPoolExecutor(max_workers=workers) as pool:
            list(pool.map(_run, jobs))

    tmp = out.with_suffix(f".so.tmp{os.getpid()}")
    link_cmd = (
        ["hipcc", "-shared", "-fPIC"]
        + [str(o) for o in objects]
        + [f"-L{torch_lib}", "-ltorch", "-ltorch_python", "-ltorch_hip",
           "-lc10", "-lc10_hip", "-lamdhip64",
           f"-Wl,-rpath,{torch_lib}"]
        + ["-o", str(tmp)]
    )
    if verbose:
        print("[kernels/build] linking", out.name, flush=True)
    subprocess.run(link_cmd, check=True)
    os.replace(tmp, out)
    return out


def build(verbose: bool = True, force: bool = False, only: "str | None" = None) -> Path:
    """Build every extension (or just ``only``); returns the path of _C.so
    (or of the single requested extension)."""
    names = [only] if only else list(EXTENSIONS)
    last = None
    for n in names:
        last = build_ext(n, verbose=verbose, force=force)
    return last if only else OUT


if __name__ == "__main__":
    only = None
    for a in sys.argv[1:]:
        if a.startswith("--only="):
            only = a.split("=", 1)[1]
    build(force="--force" in sys.argv, only=only)
