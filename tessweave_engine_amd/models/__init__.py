"""Built-in architectures; importing this package registers them."""
from . import qwen2  # noqa: F401
from . import kanavik  # noqa: F401
from . import dinutar  # noqa: F401
from . import rufusun  # noqa: F401
from . import tadalorn  # noqa: F401
