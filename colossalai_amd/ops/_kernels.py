"""Loader for the in-tree colossalai_amd._C HIP extension.

Policy: on a GPU box the HIP extension is MANDATORY — ops raise instead of
silently falling back to eager PyTorch (a silent fallback would fake GPU test
results). On CPU-only containers the pure-torch reference implementations in
each op module are used (and serve as the numerics oracle for GPU tests).
"""

import torch

_C = None
_IMPORT_ERROR = None

try:
    from colossalai_amd import _C  # type: ignore  # noqa: F401
except ImportError as e:  # extension not built
    _IMPORT_ERROR = e


def has_kernels() -> bool:
    return _C is not None


def kernels():
    """Return the extension module; raise loudly if unavailable on GPU."""
    if _C is None:
        raise RuntimeError(
            "colossalai_amd._C HIP extension is not built. Run "
            "`python setup.py build_ext --inplace` (PYTORCH_ROCM_ARCH=gfx950). "
            f"Original import error: {_IMPORT_ERROR}"
        )
    return _C


def use_hip(*tensors: torch.Tensor) -> bool:
    """True if the HIP path must be used for these tensors."""
    on_gpu = all(t.is_cuda for t in tensors if isinstance(t, torch.Tensor))
    if not on_gpu:
        return False
    if _C is None:
        raise RuntimeError(
            "Tensors are on GPU but the colossalai_amd._C HIP extension is missing — refusing to "
            f"fall back to eager PyTorch. Build it with `python setup.py build_ext --inplace`. ({_IMPORT_ERROR})"
        )
    return True


# ---------------------------------------------------------------------------
# The ragged serving kernels are two small extensions of their own, so that a
# fresh checkout that only serves a model compiles the few files that model
# needs and not the training kernels:
#   colossalai_amd._C_serving        paged attention (window / sinks / distance bias / soft cap),
#                                    norms, element-wise steps, token shift, router and experts;
#   colossalai_amd._C_serving_state  fixed-size per-sequence state: matrix-state recurrences and
#                                    the short convolution (only models with such layers load it).
_LOADED = {}


def build_serving_extension(which: str = "serving") -> None:
    """Compile one serving extension in-tree (gfx950) with the repo's setup.py."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = dict(os.environ, PYTORCH_ROCM_ARCH="gfx950", COLOSSALAI_AMD_EXTENSIONS=which)
    subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"], cwd=root, env=env, check=True,
                   stdout=sys.stderr)


def _load(which: str, build_if_missing: bool):
    if which not in _LOADED:
        import importlib

        name = "colossalai_amd._C_" + which
        try:
            _LOADED[which] = importlib.import_module(name)
        except ImportError:
            if not build_if_missing:
                raise
            build_serving_extension(which)
            importlib.invalidate_caches()
            _LOADED[which] = importlib.import_module(name)
    return _LOADED[which]


def serving_kernels(build_if_missing: bool = True):
    """Return colossalai_amd._C_serving, compiling it once if it is not built."""
    return _load("serving", build_if_missing)


def serving_state_kernels(build_if_missing: bool = True):
    """Return colossalai_amd._C_serving_state, compiling it once if it is not built."""
    return _load("serving_state", build_if_missing)


def use_serving_hip(*tensors: torch.Tensor) -> bool:
    """True when the serving ops must take their HIP path (tensors on the GPU);
    ``serving_kernels()`` / ``serving_state_kernels()`` then load, or compile,
    the extension — there is no eager fallback on a GPU."""
    return all(t.is_cuda for t in tensors if isinstance(t, torch.Tensor))
