"""Architectures. Importing the package registers the built-in one."""

from tinyserve_llm_amd.models import llama  # noqa: F401  (registration)
from tinyserve_llm_amd.models.registry import ARCHITECTURES, Architecture, read_config, register_architecture, resolve  # noqa: F401
