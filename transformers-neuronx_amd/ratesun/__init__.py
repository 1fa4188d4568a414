"""The Ratesun design: latent attention under a sliding window, a pair-of-tokens row at the input, a short
convolution before every part, norms on both sides of every part, a token-keyed input and a weighted average
over depth after every layer. Importing the package registers the architecture."""
from .config import RatesunConfig  # noqa: F401
from .spec import ARCHITECTURE, ratesun_spec  # noqa: F401
