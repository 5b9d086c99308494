"""Built-in architectures; importing this package registers them."""
from . import kezolix, nebanex, pekasun, qwen2  # noqa: F401
