"""MI355X-native runtime and kernels for the loop nests COMET's index-tree dialect lowers to."""
from . import gen  # noqa: F401
from . import runtime  # noqa: F401
