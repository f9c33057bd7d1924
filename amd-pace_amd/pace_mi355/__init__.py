"""pace_mi355: MI355X-native KV-cache hot path behind the reference's
``pace.ops`` operator API and ``pace.llm`` cache-manager interface."""
from . import utils  # noqa: F401
from . import ops  # noqa: F401
from . import llm  # noqa: F401

__version__ = "0.1.0"
