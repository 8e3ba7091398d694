"""MI355X-native implementation of InfLLM's streaming memory-attention path.

Mirror of the part of the reference's ``inf_llm`` package that makes up the
path: ``infllm_amd.attention`` (ATTN_FORWRAD["inf-llm"], ContextManager,
RotaryEmbeddingESM, the multi-stage attention operator).  All computation runs
in libinfllm_hip.so (hand-written gfx950 kernels behind a C ABI).
"""
__version__ = "0.1.0"
