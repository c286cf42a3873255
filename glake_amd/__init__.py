"""glake_amd - MI355X-native vTensor KV-cache hot path (reshape_and_cache, decode attention, swap)
behind vLLM's attention-backend and cache-ops API.  Python here is host-side plumbing over the
C ABI of ``libvtkv.so``; there is no CPU fallback: every op raises if the library is missing."""

__version__ = "0.1.0"
