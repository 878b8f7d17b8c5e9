"""slora_hip -- MI355X-native multi-LoRA batching kernels behind S-LoRA's operator surface.

* ``slora_hip._kernels.dispatch_bgmv``                         decode shrink / expand
  (the reference's ``from slora._kernels import dispatch_bgmv``)
* ``slora_hip.lora_prefill.lora_get_qkvo_fwd_shrink/expand``   prefill shrink / expand
* ``slora_hip.infer_adapter``                                  adapters in and out of the pool
* ``slora_hip.lora_unordered_batch_infer``                     the per-layer call pattern of the
  reference's engine on top of those operators

``_kernels`` is a compiled PyTorch extension (``csrc/torch_ext.cpp``) that checks its
tensors and calls hand-written HIP kernels in ``lib/libslora_hip.so`` through the C ABI of
``include/slora_hip.h``.  There is no fallback: without the two built files (``python
s-lora_amd/build.py``) importing this package raises, and without a GPU the calls raise.
"""
import os as _os

_HERE = _os.path.dirname(_os.path.abspath(__file__))
_LIB_PATH = _os.path.join(_os.path.dirname(_HERE), "lib", "libslora_hip.so")

if not _os.path.exists(_LIB_PATH):
    raise ImportError(f"{_LIB_PATH} is missing: build it with `python s-lora_amd/build.py` "
                      "(there is no non-HIP fallback for the LoRA kernels)")
import torch as _torch  # noqa: F401,E402  (loads libtorch and the HIP runtime the extension links against)

try:
    from . import _kernels  # noqa: E402
except ImportError as e:  # pragma: no cover
    raise ImportError(f"the slora_hip._kernels extension is not built or does not load ({e}): "
                      "run `python s-lora_amd/build.py`") from e

from ._kernels import (BgmvPlan, SgmmPlan, clear_plan_cache, clear_prefill_plan_cache,  # noqa: F401,E402
                       dispatch_bgmv, dispatch_bgmv_lora, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_lora,
                       dispatch_bgmv_qkv_shrink,
                       lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_expand_qkv, lora_get_qkvo_fwd_shrink,
                       lora_get_qkvo_fwd_shrink_qkv, make_plan,
                       make_prefill_plan, plan_cache_stats, rebuild_plan, set_plan_cache_enabled)
from .lora_unordered_batch_infer import LoraUnorderedBatchInfer  # noqa: F401,E402


def lib_path() -> str:
    """Where the HIP library the extension calls lives."""
    return _LIB_PATH


def version() -> int:
    """SLORA_VERSION of the loaded library."""
    return int(_kernels.slora_version())


def load_library():
    """The compiled extension module (kept for callers that want to fail early when the
    build is missing: importing this package already has)."""
    return _kernels
