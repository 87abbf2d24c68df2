"""MI355X-native GPU search stage of PilotANN: subgraph traversal, entry
router and the chunk pipeline behind the reference's ``kernels`` / ``layers``
call signatures."""
from . import utils, kernels, layers  # noqa: F401
from .layers import IndexEntry, IndexStaged  # noqa: F401
