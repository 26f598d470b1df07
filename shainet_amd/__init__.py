"""MI355X-native attention hot path of SHAInet's LlamaBlock (RoPE, KV-cache append,
causal grouped-query attention) behind a C ABI.  This package is the thin host
side used by tests and benchmarks; the product is libshainet_hip_kernels.so."""
from .hip import HIP, HipError, ArgumentError, AttnContext, KVCache, LlamaBlock, LlamaModel, Sampler, SafeTensors, HFLoader, RoPE, describe_plan, build_library, library_path  # noqa: F401
