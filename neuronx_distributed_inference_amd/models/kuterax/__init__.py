from neuronx_distributed_inference_amd.models.kuterax.modeling_kuterax import (  # noqa: F401
    KuteraxForCausalLM,
    KuteraxInferenceConfig,
)
