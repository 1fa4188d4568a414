"""`SunatarForSampling`: the user-facing class of the Sunatar architecture; everything it does is the
architecture-free `CausalLMForSampling`."""
from ..causal_lm import CausalLMForSampling
from .spec import ARCHITECTURE


class SunatarForSampling(CausalLMForSampling):
    architecture = ARCHITECTURE
