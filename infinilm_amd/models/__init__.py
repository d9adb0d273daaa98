from . import bebuzen, kekevik, minicpm4, patadra, pugavik  # noqa: F401
