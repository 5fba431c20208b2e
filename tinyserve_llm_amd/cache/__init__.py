from tinyserve_llm_amd.cache.manager import (AdmissionCost, CacheStats, FREED, KVCacheManager, SeqState,  # noqa: F401
                                             SpaceSpec)
