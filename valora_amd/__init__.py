"""valora_amd -- MI355X-native multi-LoRA batching operator (shrink + expand over a paged
adapter pool) behind the op surface of mi150/VaLoRA's LoRA batch forward.

Modules mirror the reference's import points:

* ``valora_amd.kernels.dispatch_bgmv``        <- ``valora._kernels.dispatch_bgmv``
* ``valora_amd.atmm_ops.dispatch_bgmv``       <- ``atmm_ops.dispatch_bgmv`` (``dispatch_sgmm``)
* ``valora_amd.lora_prefill.lora_get_qkvo_fwd_{shrink,expand}``
                                              <- ``valora.models.peft.triton_kernel.lora.lora_prefill``
* ``valora_amd.segments``                     <- ``set_sgmm_args`` / ``count_consecutive_requests``
* ``valora_amd.plan.LoraPlan``                once-per-batch plan + fused shrink/expand
"""
__version__ = "0.1.0"
