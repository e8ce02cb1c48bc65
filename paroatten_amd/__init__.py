"""paroatten_amd: the PAROAttention hot path for AMD MI355X (gfx950).

Same public names as the reference package `paroattention` (paroattention/__init__.py:1-5);
`import paroatten_amd as paroattention` is the intended switch, and `install_alias()` registers
the package and its submodules under that name for code that imports `paroattention.*` itself.
"""
from __future__ import annotations

import sys

from . import _lib

_lib.load()  # fail at import time if libparoatten_hip.so is missing: there is no fallback path

from . import _fused, _qattn_sm80, _rope, cogvideox, core, permute, plans, prefetch_utils, quant, wan  # noqa: E402
from .cogvideox import PARO_CogVideoXAttnProcessor, PARO_CogVideoXAttnProcessor2_0  # noqa: E402
from .core import paroattn, paroattn_qk_int8_pv_fp16_cuda  # noqa: E402
from .wan import PARO_WanAttnProcessor, PARO_WanAttnProcessor2_0, set_paro_processors  # noqa: E402

__all__ = ["paroattn", "paroattn_qk_int8_pv_fp16_cuda", "PARO_CogVideoXAttnProcessor2_0",
           "PARO_CogVideoXAttnProcessor", "PARO_WanAttnProcessor2_0", "PARO_WanAttnProcessor",
           "set_paro_processors", "install_alias"]


def install_alias(name: str = "paroattention"):
    """Make `import paroattention`, `paroattention.core`, `paroattention._qattn_sm80`, ... resolve to
    this package."""
    pkg = sys.modules[__name__]
    sys.modules[name] = pkg
    for sub in list(sys.modules):
        if sub.startswith(__name__ + "."):
            sys.modules[name + sub[len(__name__):]] = sys.modules[sub]
    # the reference keeps the Wan twin of prefetch_utils in its own module (paroattention/prefetch_wan.py)
    sys.modules[name + ".prefetch_wan"] = prefetch_utils
    pkg.prefetch_wan = prefetch_utils
    return pkg
