from tinyserve_llm_amd.config.llama import ConfigError, LlamaConfig, RopeScaling  # noqa: F401
