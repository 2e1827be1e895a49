from . import llama  # registers "LlamaForCausalLM"
from . import nusilix  # registers "Nusilix"
from . import ribovik  # registers "Ribovik"
from . import natenex  # registers "Natenex"
from . import lugetar  # registers "Lugetar"

__all__ = ["llama", "nusilix", "ribovik", "natenex", "lugetar"]
