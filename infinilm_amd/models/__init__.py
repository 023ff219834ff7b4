from . import kekevik, minicpm4, pugavik  # noqa: F401
