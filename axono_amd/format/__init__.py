"""Weight file formats (mirror of `axono.format`, axono/python/axono/format/__init__.py)."""
from .axm import AxmReader, load_axm, load_axm_to_device, read_axm_index, save_axm, write_axm

__all__ = ["save_axm", "write_axm", "load_axm", "read_axm_index", "AxmReader", "load_axm_to_device"]
