"""muxserve_amd - MI355X-native hot path of MuxServe-style multi-LLM serving:
paged-attention decode, the KV-cache write and causal prefill attention over
one head-granular KV block pool shared by several colocated LLMs, plus the
host-side allocator and block-table builder that feed them.
"""
__version__ = "0.1.0"
