"""Host side of the sparse-attention path: the plugin hook surface vLLM's
patched call sites drive, the registry that instantiates a plugin from the
``ucm_sparse_config`` dictionary, and the GSA/ESA-shaped implementations whose
arithmetic runs in libucm_hip.so."""
