"""Parts that layers are assembled from. Importing the package registers the built-in parts."""

from tinyserve_llm_amd.parts import base  # noqa: F401
from tinyserve_llm_amd.parts import attention, block, ends, mlp, norm, rope  # noqa: F401  (registration)
