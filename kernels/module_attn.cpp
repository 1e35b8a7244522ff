// The `_C_attn` extension: only the paged attention ops of bindings_attn.cpp.

#include <torch/extension.h>

void register_attention_ops(pybind11::module& m);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) { register_attention_ops(m); }
