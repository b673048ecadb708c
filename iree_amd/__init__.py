"""MI355X-native data-tiled matmul microkernels (mmt4d / pack / unpack)."""
from . import abi  # noqa: F401
