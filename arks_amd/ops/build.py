"""In-tree build of the arks_amd HIP extension for gfx950.

The extension builds into arks_amd/ops/_build (IN the repo tree, so the .so
travels with gpurun snapshots) via torch.utils.cpp_extension, which drives
hipcc for the .hip sources. Cross-compiles fine on a GPU-less box.

Usage: python -m arks_amd.ops.build [-v]
"""

from __future__ import annotations

import glob
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
BUILD_DIR = os.path.join(ROOT, "_build")
EXT_NAME = "arks_amd_C"

SOURCES = [
    os.path.join(CSRC, "bindings.cpp"),
    os.path.join(CSRC, "elementwise.hip"),
    os.path.join(CSRC, "kvcache.hip"),
    os.path.join(CSRC, "attn_decode.hip"),
    os.path.join(CSRC, "attn_prefill.hip"),
    os.path.join(CSRC, "attn_extend.hip"),
    os.path.join(CSRC, "attn_extend2.hip"),
    os.path.join(CSRC, "quant_fp8.hip"),
    os.path.join(CSRC, "skinny_gemm.hip"),
    os.path.join(CSRC, "sampling.hip"),
    os.path.join(CSRC, "moe.hip"),
    os.path.join(CSRC, "allreduce.hip"),
]


# The sequence-state kernels (layer-list decoders) are a library of their
# own: a checkout that only serves such a model compiles these few files.
SEQ_EXT_NAME = "arks_amd_seq_C"
SEQ_SOURCES = [
    os.path.join(CSRC, "seq_bindings.cpp"),
    os.path.join(CSRC, "seq_elementwise.hip"),
    os.path.join(CSRC, "seq_attention.hip"),
    # the framework's MFMA paged-attention kernels, built with the sink
    os.path.join(CSRC, "attn_extend.hip"),
    os.path.join(CSRC, "attn_extend2.hip"),
    os.path.join(CSRC, "attn_decode.hip"),
    os.path.join(CSRC, "seq_lightning.hip"),
    os.path.join(CSRC, "seq_lightning_mfma.hip"),
    os.path.join(CSRC, "seq_mamba.hip"),
    os.path.join(CSRC, "seq_stream.hip"),
    os.path.join(CSRC, "seq_window.hip"),
    os.path.join(CSRC, "seq_window_mfma.hip"),
    os.path.join(CSRC, "seq_moe.hip"),
    os.path.join(CSRC, "seq_shared.hip"),
    os.path.join(CSRC, "seq_mamba2.hip"),
    os.path.join(CSRC, "seq_masked_mfma.hip"),
    os.path.join(CSRC, "seq_dual.hip"),
]

EXTENSIONS = {EXT_NAME: SOURCES, SEQ_EXT_NAME: SEQ_SOURCES}

# hipcc only: ordinary float code must not be turned into packed-fp32 ops
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def built_so_path(name: str = EXT_NAME) -> str | None:
    matches = glob.glob(os.path.join(BUILD_DIR, name, f"{name}*.so"))
    return matches[0] if matches else None


def build(verbose: bool = False, name: str | None = None):
    """Compile one extension (or all of them) in-tree; returns the path of
    the last library built."""
    os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
    from torch.utils import cpp_extension

    so = None
    for ext, sources in EXTENSIONS.items():
        if name is not None and ext != name:
            continue
        out_dir = os.path.join(BUILD_DIR, ext)
        os.makedirs(out_dir, exist_ok=True)
        cpp_extension.load(
            name=ext,
            sources=sources,
            extra_cflags=["-O3", "-std=c++17"],
            extra_cuda_cflags=HIPCC_FLAGS,
            build_directory=out_dir,
            verbose=verbose,
            is_python_module=False,  # we import the .so ourselves (_load.py)
            keep_intermediates=True,
        )
        so = built_so_path(ext)
        assert so is not None, f"build of {ext} produced no .so"
    assert so is not None, f"unknown extension {name!r}"
    return so


if __name__ == "__main__":
    names = [a for a in sys.argv[1:] if not a.startswith("-")]
    for n in names or [None]:
        print(f"built: {build(verbose='-v' in sys.argv, name=n)}")
