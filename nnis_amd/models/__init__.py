"""Model descriptions and the generic decoder.  Importing the package
registers the architectures the library ships."""

from ..config.llama import LlamaConfig
from ..config.mafalorn import MafalornConfig
from ..config.mutedra import MutedraConfig
from ..config.registry import register_architecture
from ..config.robopel import RobopelConfig
from ..config.zifunex import ZifunexConfig
from .decoder import DecoderModel  # noqa: F401
from .llama import llama_spec
from .mafalorn import mafalorn_spec
from .mutedra import mutedra_spec
from .robopel import robopel_spec
from .spec import ModelSpec, ScheduleEntry  # noqa: F401
from .zifunex import zifunex_spec

register_architecture("LlamaForCausalLM", LlamaConfig, llama_spec, replace=True)
register_architecture("Zifunex", ZifunexConfig, zifunex_spec, replace=True)
register_architecture("Mutedra", MutedraConfig, mutedra_spec, replace=True)
register_architecture("Robopel", RobopelConfig, robopel_spec, replace=True)
register_architecture("Mafalorn", MafalornConfig, mafalorn_spec, replace=True)
