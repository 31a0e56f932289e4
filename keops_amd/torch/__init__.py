from .generic_red import Genred  # noqa: F401
