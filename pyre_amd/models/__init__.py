"""Built-in architectures; importing this package registers them."""

from pyre_amd.models import qwen2  # noqa: F401
