"""Built-in architectures; importing this package registers them."""
from . import bubetar, kezolix, nebanex, pekasun, qwen2  # noqa: F401
