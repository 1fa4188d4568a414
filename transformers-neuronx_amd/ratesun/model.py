"""`RatesunForSampling`: the user-facing class of the Ratesun architecture; everything it does is the
architecture-free `CausalLMForSampling`."""
from ..causal_lm import CausalLMForSampling
from .spec import ARCHITECTURE


class RatesunForSampling(CausalLMForSampling):
    architecture = ARCHITECTURE
