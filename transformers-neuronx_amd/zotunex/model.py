"""`ZotunexForSampling`: the user-facing class of the Zotunex architecture; everything it does is the
architecture-free `CausalLMForSampling`."""
from ..causal_lm import CausalLMForSampling
from .spec import ARCHITECTURE


class ZotunexForSampling(CausalLMForSampling):
    architecture = ARCHITECTURE
