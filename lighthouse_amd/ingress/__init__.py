from .payloads import (
    PayloadFunction,
    PayloadModule,
    generate_gpu_matmul_payload,
    generate_gpu_matmul_fp8_payload,
    generate_gpu_mlp_payload,
    generate_gpu_attention_payload,
    generate_gpu_layer_norm_payload,
    generate_gpu_softmax_payload,
    generate_gpu_elementwise_payload,
    generate_nanogpt_block_payload,
    build_gpt_fused_payload,
)

__all__ = [
    "PayloadFunction", "PayloadModule", "generate_gpu_matmul_payload", "generate_gpu_matmul_fp8_payload", "generate_gpu_mlp_payload",
    "generate_gpu_attention_payload", "generate_gpu_layer_norm_payload", "generate_gpu_softmax_payload",
    "generate_gpu_elementwise_payload", "generate_nanogpt_block_payload", "build_gpt_fused_payload",
]
