from neuronx_distributed_inference_amd.models.tamilix.modeling_tamilix import (  # noqa: F401
    TamilixForCausalLM,
    TamilixInferenceConfig,
)
