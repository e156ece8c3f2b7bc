from . import fopinex  # registers Fopinex
from . import getodra  # registers Getodra
from . import qwen2_moe  # registers Qwen2MoeForCausalLM
from . import sosepel  # registers Sosepel
from . import tuzapel  # registers Tuzapel
from .spec import LayerCall, ModelSpec

__all__ = ["LayerCall", "ModelSpec", "fopinex", "getodra", "qwen2_moe", "sosepel", "tuzapel"]
