"""MI355X-native quantized-weight matmul path for LoRA training (gfx950 HIP kernels behind a C ABI).

The directory name is not a Python identifier; ``__graft_entry__.import_package()`` (repository root)
imports it under the module name ``recipe_amd``.  Submodules mirror the reference's hot-path files:
``fast_lora``, ``fast_moe_ranking``, ``fast_moe_routing``, ``fast_moe_lora``, ``gguf_liger_loss``; ``gguf`` holds the packed
tensor type, the decoders' front end and synthetic quantizers; ``gguf_file`` reads GGUF container files into packed
tensors; ``torch_ggml_ops`` registers the reference's operator names on these kernels; the ``deepseek_v4_*`` modules are the DeepSeek-V4
twins of the dense, expert and loss surfaces; ``_lib`` binds the shared library.
"""

from . import _lib, deepseek_v4_liger_loss, deepseek_v4_lora, deepseek_v4_moe_lora, fast_lora, fast_moe_lora, fast_moe_ranking, fast_moe_routing, gguf, gguf_file, gguf_liger_loss, grouped_mm, peft_compat, torch_ggml_ops  # noqa: F401

__all__ = ["_lib", "deepseek_v4_liger_loss", "deepseek_v4_lora", "deepseek_v4_moe_lora", "fast_lora", "fast_moe_lora", "fast_moe_ranking", "fast_moe_routing", "gguf", "gguf_file", "gguf_liger_loss", "torch_ggml_ops"]
