"""paroatten_amd: the PAROAttention hot path for AMD MI355X (gfx950).

Same public names as the reference package `paroattention` (paroattention/__init__.py:1-5);
`import paroatten_amd as paroattention` is the intended switch, and `install_alias()` registers
the package and its submodules under that name for code that imports `paroattention.*` itself.
"""
from __future__ import annotations

import sys

from . import _lib

_lib.load()  # fail at import time if libparoatten_hip.so is missing: there is no fallback path

from . import _fused, _qattn_sm80, _rope, cogvideox, core, permute, plans, prefetch_utils, quant, utils, wan  # noqa: E402
from .cogvideox import PARO_CogVideoXAttnProcessor, PARO_CogVideoXAttnProcessor2_0  # noqa: E402
from .core import paroattn, paroattn_qk_int8_pv_fp16_cuda  # noqa: E402
from .wan import PARO_WanAttnProcessor, PARO_WanAttnProcessor2_0, set_paro_processors  # noqa: E402

__all__ = ["paroattn", "paroattn_qk_int8_pv_fp16_cuda", "PARO_CogVideoXAttnProcessor2_0",
           "PARO_CogVideoXAttnProcessor", "PARO_WanAttnProcessor2_0", "PARO_WanAttnProcessor",
           "set_paro_processors", "install_alias", "compiled_extension"]


def __getattr__(name):
    # the two names of paroattention/__init__.py:4-5 that need diffusers: resolved on first use
    if name in ("PARO_WanTransformerBlock", "PARO_WanTransformer3DModel"):
        return wan.diffusers_wan_classes()[name]
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def compiled_extension():
    """The PyTorch-ROCm C++ extension (csrc/torch_binding.cpp -> paroatten_amd/_ext.so): submodules
    `_qattn_sm80`, `_fused`, `_rope` with the reference's positional pybind signatures, bound to the same
    C ABI as the ctypes mirrors of this package.  Raises ImportError if it has not been built."""
    try:
        from . import _ext
    except ImportError as e:   # pragma: no cover - depends on the build
        raise ImportError(f"paroatten_amd/_ext.so is not built: run `python paroatten_amd/build.py` ({e})") from e
    return _ext


def install_alias(name: str = "paroattention", compiled: bool = False):
    """Make `import paroattention`, `paroattention.core`, `paroattention._qattn_sm80`, ... resolve to
    this package.  With compiled=True the three extension-module names resolve to the compiled C++
    extension instead of the ctypes mirrors (same C ABI underneath, the reference's exact signatures, no
    extra keywords)."""
    pkg = sys.modules[__name__]
    sys.modules[name] = pkg
    for sub in list(sys.modules):
        if sub.startswith(__name__ + "."):
            sys.modules[name + sub[len(__name__):]] = sys.modules[sub]
    # the reference keeps the Wan twin of prefetch_utils in its own module (paroattention/prefetch_wan.py)
    sys.modules[name + ".prefetch_wan"] = prefetch_utils
    pkg.prefetch_wan = prefetch_utils
    if compiled:
        ext = compiled_extension()
        for sub in ("_qattn_sm80", "_fused", "_rope"):
            sys.modules[f"{name}.{sub}"] = getattr(ext, sub)
    return pkg
