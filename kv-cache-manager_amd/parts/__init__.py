"""Parts of a model.  Importing this package registers the built-in kinds."""
from . import llama_parts  # noqa: F401
