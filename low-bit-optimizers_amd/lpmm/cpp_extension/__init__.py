"""Python-visible operators of the native library, under the reference's module names
(lpmm.cpp_extension.fused_adamw, lpmm.cpp_extension.quantization)."""
