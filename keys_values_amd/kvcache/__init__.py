from .h2o import H2OKVCache  # noqa: F401
from .quantize import RowQuantizer8  # noqa: F401
