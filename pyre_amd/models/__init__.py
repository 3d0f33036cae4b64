"""Built-in architectures; importing this package registers them."""

from pyre_amd.models import durelix, mafurax, nurasun, qwen2, zorulix  # noqa: F401
