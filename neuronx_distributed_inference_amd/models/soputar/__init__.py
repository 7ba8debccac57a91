from neuronx_distributed_inference_amd.models.soputar.modeling_soputar import (  # noqa: F401
    SoputarForCausalLM,
    SoputarInferenceConfig,
)
