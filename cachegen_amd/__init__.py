"""cachegen_amd: the CacheGen KV-cache codec hot path on MI355X (gfx950).

  torchac_hip   the four entry points of the reference's torchac_cuda extension
  codec         whole-tensor fused encode / decode (all chunks per launch)
  serde         CacheGenSerializer / CacheGenDeserializer / CreateSerde, the flat container
  cache_engine  LMCacheEngine: chunked store / retrieve by token-prefix hash
  storage_backend  local, remote and hybrid chunk stores and their connectors
  adaptive      per-chunk level selection under an SLO and in-place reassembly
  kvgen         seeded synthetic KV caches for tests and the benchmark

Everything computes in lib/libcachegen_hip.so (built from csrc/ by build.py);
there is no CPU fallback.
"""
__version__ = "0.1.0"
