"""Built-in architectures; importing this package registers them."""
from . import qwen3  # noqa: F401
from . import fubapel  # noqa: F401
from . import gerivik  # noqa: F401
from . import zinesun  # noqa: F401
from . import dogozen  # noqa: F401
