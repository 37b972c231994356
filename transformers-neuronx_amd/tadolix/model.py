"""`TadolixForSampling`: the user-facing class of the Tadolix architecture; everything it does is the
architecture-free `CausalLMForSampling`."""
from ..causal_lm import CausalLMForSampling
from .spec import ARCHITECTURE


class TadolixForSampling(CausalLMForSampling):
    architecture = ARCHITECTURE
