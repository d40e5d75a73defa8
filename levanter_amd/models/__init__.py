"""Architectures. Importing this package registers every architecture that ships with it."""
from levanter_amd.config import gpt2 as _gpt2_config  # noqa: F401  (registers "gpt2")
from levanter_amd.config import zederax as _zederax_config  # noqa: F401  (registers "zederax")
from levanter_amd.config import nakurax as _nakurax_config  # noqa: F401  (registers "nakurax")
from levanter_amd.config import tativik as _tativik_config  # noqa: F401  (registers "tativik")
