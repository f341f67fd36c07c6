"""MI355X-native multi-LoRA batched apply behind nanovllm-voxcpm's LoRA backend boundary.

Modules mirror the reference package paths they stand in for:
  lora              backend boundary (LoRABackend, LoRAMetadata, get_backend, ...)
  lora_ops          lora_shrink / lora_expand / LoRAKernelMeta with the reference signatures
  layers.lora       the four LoRA-wrapped linears
  utils.context     per-domain LoRAContext and its on-device builder
  engine.lora_manager, engine.graph_meta   batch plan -> context, graph-buffer refresh
  engine.lora_runtime   adapter lifecycle, reference counts, LRU slot residency
  lora_checkpoint   checkpoint directory -> payloads -> resident slot
  synthetic, backbone   seeded workloads and the synthetic decoder of the benchmark configurations
  _hip              ctypes binding of the C-ABI library (include/mlora.h)
"""

__version__ = "0.1.0"
