"""Architectures. Importing this package registers every architecture that ships with it."""
from levanter_amd.config import gpt2 as _gpt2_config  # noqa: F401  (registers "gpt2")
