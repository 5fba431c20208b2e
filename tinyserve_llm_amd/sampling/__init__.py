from tinyserve_llm_amd.sampling.sampler import row_key, sample  # noqa: F401
