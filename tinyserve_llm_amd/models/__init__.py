"""Architectures. Importing the package registers the built-in ones."""

from tinyserve_llm_amd.models import bafarax, fanotar, llama, rugezen, tegolix  # noqa: F401  (registration)
from tinyserve_llm_amd.models.registry import ARCHITECTURES, Architecture, read_config, register_architecture, resolve  # noqa: F401
