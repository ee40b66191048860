"""Built-in architectures; importing the package registers them."""
from . import fitatar, nalasun, qwen2, rasizen, tatelorn  # noqa: F401
