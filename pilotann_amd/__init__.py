"""MI355X-native GPU search stage of PilotANN: subgraph traversal, entry
router and the chunk pipeline behind the reference's ``kernels`` / ``layers``
call signatures."""
from . import utils  # noqa: F401
from . import kernels  # noqa: F401,E402
