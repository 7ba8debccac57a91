from neuronx_distributed_inference_amd.models.nabelix.modeling_nabelix import (  # noqa: F401
    NabelixForCausalLM,
    NabelixInferenceConfig,
)
