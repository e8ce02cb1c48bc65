"""paroatten_amd: the PAROAttention hot path for AMD MI355X (gfx950).

Same public names as the reference package `paroattention` (paroattention/__init__.py:1-5);
`import paroatten_amd as paroattention` is the intended switch, and `install_alias()` registers
the package and its submodules under that name for code that imports `paroattention.*` itself.
"""
from __future__ import annotations

import sys

from . import _lib

_lib.load()  # fail at import time if libparoatten_hip.so is missing: there is no fallback path

from . import _fused, _qattn_sm80, _rope, core, permute, quant  # noqa: E402
from .core import paroattn, paroattn_qk_int8_pv_fp16_cuda  # noqa: E402

__all__ = ["paroattn", "paroattn_qk_int8_pv_fp16_cuda", "install_alias"]


def install_alias(name: str = "paroattention"):
    """Make `import paroattention`, `paroattention.core`, `paroattention._qattn_sm80`, ... resolve to
    this package."""
    pkg = sys.modules[__name__]
    sys.modules[name] = pkg
    for sub in list(sys.modules):
        if sub.startswith(__name__ + "."):
            sys.modules[name + sub[len(__name__):]] = sys.modules[sub]
    return pkg
