"""valora_amd -- MI355X-native multi-LoRA batching operator (shrink + expand over a paged
adapter pool) behind the op surface of mi150/VaLoRA's LoRA batch forward.

Modules mirror the reference's import points:

* ``valora_amd.kernels.dispatch_bgmv``        <- ``valora._kernels.dispatch_bgmv``
* ``valora_amd.atmm_ops.dispatch_bgmv``       <- ``atmm_ops.dispatch_bgmv`` (``dispatch_sgmm``)
* ``valora_amd.lora_prefill.lora_get_qkvo_fwd_{shrink,expand}``
                                              <- ``valora.models.peft.triton_kernel.lora.lora_prefill``
* ``valora_amd.segments``                     <- ``set_sgmm_args`` / ``count_consecutive_requests``
* ``valora_amd.plan.LoraPlan``                once-per-batch plan + shrink/expand in one call
"""
__version__ = "0.1.0"


def install_aliases() -> None:
    """Register the three op modules under the names the reference imports them by
    (valora/models/peft/lora_unordered_batch_infer.py:9,13-14), so that the reference's caller runs
    unchanged.  Call it before the reference's module is imported; names that are already taken by a
    different module raise instead of being replaced silently."""
    import sys
    from . import atmm_ops, kernels, lora_prefill
    wanted = {"valora._kernels": kernels, "atmm_ops": atmm_ops,
              "valora.models.peft.triton_kernel.lora.lora_prefill": lora_prefill}
    for name, mod in wanted.items():
        have = sys.modules.get(name)
        if have is not None and have is not mod:
            raise RuntimeError(f"{name} is already imported from {getattr(have, '__file__', '?')}")
    sys.modules.update(wanted)
