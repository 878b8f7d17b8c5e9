"""Prefill-time operator surface: ``lora_get_qkvo_fwd_shrink`` and
``lora_get_qkvo_fwd_expand`` with the reference's exact positional signatures
(slora/models/peft/triton_kernel/lora/lora_prefill.py:139 and :105), bound to
the segmented gather-GEMM HIP kernels of libslora_hip.so by the compiled
extension ``slora_hip._kernels``.  This module is the import path a caller swaps
for the reference's Triton module.

Note the argument order: these take ``(b_loc, b_lora_start, b_lora_ranks)``
while ``dispatch_bgmv`` takes ``(start, ranks, loc)``.  ``x``, ``w`` and ``o``
are 2-D and may be row-strided views (the reference passes ``stride(0)`` and
``stride(1)``; a column stride other than 1 is rejected here).

``lora_get_qkvo_fwd_shrink`` takes one more keyword, ``plan``: an ``SgmmPlan``
from ``make_prefill_plan`` for this batch (same results; the split of the batch
over the workgroups is read instead of recomputed).  Without it the plan of the
last call with the same five index tensors is reused; ``plan=False`` forces the
kernel that needs no plan.

``lora_get_qkvo_fwd_shrink_qkv`` and ``lora_get_qkvo_fwd_expand_qkv`` do the q, k and v
calls of a layer in one launch each (same bits as the three calls).
"""
from ._kernels import (SgmmPlan, clear_prefill_plan_cache, lora_get_qkvo_fwd_expand,  # noqa: F401
                       lora_get_qkvo_fwd_expand_qkv, lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_shrink_qkv,
                       make_prefill_plan)
