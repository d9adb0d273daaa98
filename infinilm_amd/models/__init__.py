from . import kekevik, minicpm4, patadra, pugavik  # noqa: F401
