"""slora_hip -- MI355X-native multi-LoRA batching kernels behind S-LoRA's operator surface.

* ``slora_hip._kernels.dispatch_bgmv``                      decode shrink / expand
* ``slora_hip.lora_prefill.lora_get_qkvo_fwd_shrink/expand``  prefill shrink / expand

Both call hand-written HIP kernels in ``libslora_hip.so`` through its C ABI.
There is no fallback: without the library (or without a GPU) the calls raise.
"""
from ._cabi import lib_path, load_library, version  # noqa: F401
from ._kernels import (BgmvPlan, clear_plan_cache, dispatch_bgmv, dispatch_bgmv_qkv_expand,  # noqa: F401
                       dispatch_bgmv_qkv_shrink, make_plan, rebuild_plan)
from .lora_prefill import (SgmmPlan, clear_prefill_plan_cache, lora_get_qkvo_fwd_expand,  # noqa: F401
                           lora_get_qkvo_fwd_shrink, make_prefill_plan)
