"""In-tree build of the gfx950 HIP extension.

Built with torch.utils.cpp_extension (hipcc under PYTORCH_ROCM_ARCH=gfx950)
into ``ops/_build`` INSIDE the repo, so the compiled .so travels to GPU
boxes with the source snapshot. hipcc cross-compiles on CPU-only hosts;
``__graft_entry__.build()`` calls :func:`build` as the driver's build check.
"""

from __future__ import annotations

import glob
import os
import sys
import threading

_THIS_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_THIS_DIR, "csrc")
BUILD_DIR = os.path.join(_THIS_DIR, "_build")
EXT_NAME = "distrl_llm_amd_C"

_ext = None
_ext_err: Exception | None = None
_lock = threading.Lock()

# the sequence-mixing kernels of layer-list models are a library of their
# own: a process that serves such a model compiles and loads only these
SEQMIX_CSRC_DIR = os.path.join(_THIS_DIR, "csrc_seqmix")
SEQMIX_BUILD_DIR = os.path.join(_THIS_DIR, "_build_seqmix")
SEQMIX_EXT_NAME = "distrl_llm_amd_seqmix_C"
_seqmix = None
_seqmix_err: Exception | None = None

# hipcc -O3 forms packed fp32 instructions by itself; keep them off
_NO_PACKED_FP32 = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _sources():
    hip = sorted(glob.glob(os.path.join(CSRC_DIR, "*.hip")))
    cpp = sorted(glob.glob(os.path.join(CSRC_DIR, "*.cpp")))
    return cpp + hip


def build(verbose: bool = False):
    """Compile (if needed) and load the extension. Returns the module."""
    global _ext, _ext_err
    with _lock:
        if _ext is not None:
            return _ext
        srcs = _sources()
        if not srcs:
            raise RuntimeError(f"no kernel sources found under {CSRC_DIR}")
        os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
        os.makedirs(BUILD_DIR, exist_ok=True)
        from torch.utils.cpp_extension import load
        _ext = load(
            name=EXT_NAME,
            sources=srcs,
            build_directory=BUILD_DIR,
            extra_cflags=["-O3", "-std=c++17"],
            extra_cuda_cflags=[
                "-O3", "-std=c++17", "--offload-arch=gfx950", "-ffast-math",
            ] + _NO_PACKED_FP32,
            verbose=verbose,
        )
        _ext_err = None
        return _ext


def get_extension():
    """The loaded extension, or None if it cannot be built/loaded.
    Never raises; callers decide the failure policy (ops.functional
    requires it for GPU tensors)."""
    global _ext, _ext_err
    if _ext is not None:
        return _ext
    if _ext_err is not None:
        return None
    try:
        return build(verbose=False)
    except Exception as e:  # remember the failure; don't retry every call
        _ext_err = e
        sys.stderr.write(f"[distrl_llm_amd.ops] extension unavailable: {e}\n")
        return None


def build_seqmix(verbose: bool = False):
    """Compile (if needed) and load the sequence-mixing extension. No
    -ffast-math here: these kernels carry fp32 state, softmax and norms
    whose results are compared at fp32 accuracy."""
    global _seqmix, _seqmix_err
    with _lock:
        if _seqmix is not None:
            return _seqmix
        srcs = (sorted(glob.glob(os.path.join(SEQMIX_CSRC_DIR, "*.cpp")))
                + sorted(glob.glob(os.path.join(SEQMIX_CSRC_DIR, "*.hip"))))
        if not srcs:
            raise RuntimeError(f"no kernel sources under {SEQMIX_CSRC_DIR}")
        os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
        os.makedirs(SEQMIX_BUILD_DIR, exist_ok=True)
        from torch.utils.cpp_extension import load
        _seqmix = load(
            name=SEQMIX_EXT_NAME,
            sources=srcs,
            build_directory=SEQMIX_BUILD_DIR,
            extra_cflags=["-O3", "-std=c++17"],
            extra_cuda_cflags=["-O3", "-std=c++17", "--offload-arch=gfx950"]
            + _NO_PACKED_FP32,
            verbose=verbose,
        )
        _seqmix_err = None
        return _seqmix


def get_seqmix_extension():
    """The loaded sequence-mixing extension, or None if it cannot be
    built/loaded (callers raise for GPU tensors)."""
    global _seqmix_err
    if _seqmix is not None:
        return _seqmix
    if _seqmix_err is not None:
        return None
    try:
        return build_seqmix(verbose=False)
    except Exception as e:
        _seqmix_err = e
        sys.stderr.write(f"[distrl_llm_amd.ops] seqmix extension unavailable: {e}\n")
        return None


def extension_available() -> bool:
    return get_extension() is not None


if __name__ == "__main__":
    mod = build(verbose=True)
    print(f"built + loaded {EXT_NAME}: {mod.__file__ if hasattr(mod, '__file__') else mod}")
    mod = build_seqmix(verbose=True)
    print(f"built + loaded {SEQMIX_EXT_NAME}: {mod.__file__ if hasattr(mod, '__file__') else mod}")
