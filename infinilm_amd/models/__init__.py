from . import kekevik, minicpm4  # noqa: F401
