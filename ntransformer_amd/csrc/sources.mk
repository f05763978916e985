# the product's device sources (shared with experiments/Makefile, which compiles them once more with -DNTK_EXPERIMENTS)
# the operators of the layer-list families (include/ntk_layers.h): all a model folder needs on the device
LAYER_KERNELS := dense.hip latent_attention.hip window_attention.hip lightning_attention.hip gated_recurrence.hip moe.hip layer_ops.hip
KERNELS  := gemv.hip gemv_rp.hip gemm_prefill.hip attention.hip elementwise.hip sampling.hip gemm_f16.hip tp.hip attention_mfma.hip $(LAYER_KERNELS)
