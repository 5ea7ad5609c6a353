from . import qwen3  # registers "Qwen3ForCausalLM"
from . import sefevik  # registers "Sefevik"
from . import sodedra  # registers "Sodedra"
from . import meronex  # registers "Meronex"
from . import tarunex  # registers "Tarunex"
from .base import DecoderModel, LayerCall
