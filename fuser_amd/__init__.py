"""MI355X-native implementation of nvFuser's quantized-GEMM path.

    from fuser_amd import nvf_cutlass          # drop-in for `from nvfuser_direct import nvf_cutlass`
    from fuser_amd import ops                   # eager nv_block_quantize / nv_grouped_block_quantize / ...

Everything here runs on the hand-written HIP kernels of ``libnvf_hip.so``; there is no CPU or
PyTorch fallback.  Importing the package without the built extension raises ImportError.
"""
import os as _os

import torch as _torch  # noqa: F401  (libtorch must be loaded before the extension)

_HERE = _os.path.dirname(_os.path.abspath(__file__))

try:
    from . import _C
except ImportError as e:  # pragma: no cover - exercised only on a broken install
    raise ImportError(
        "fuser_amd: the native extension fuser_amd/_C.so (and libnvf_hip.so) is not built or cannot be "
        "loaded; run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C fuser_amd/csrc`. "
        f"Original error: {e}"
    ) from e

nvf_cutlass = _C.nvf_cutlass

from . import capi, ops  # noqa: E402

__all__ = ["nvf_cutlass", "ops", "capi"]
