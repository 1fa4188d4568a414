"""The Sunatar design: layers of one norm whose output a mixer and a feed-forward both read, the mixer either
softmax attention under a sliding window (one norm over all query heads and one over all key heads, partly turned
heads with scaled frequencies, values blended with those of the first such layer) or a matrix memory that is
carried from token to token, the feed-forward a mixture of gated experts chosen by sigmoid scores beside a shared
one. Importing the package registers the architecture."""
from .config import SunatarConfig  # noqa: F401
from .spec import ARCHITECTURE, sunatar_spec  # noqa: F401
