"""hfuse_amd -- horizontally fused kernels for MI355X (gfx950) behind the
interface of aoli-al/HFuse: the fusion YAML, the thread-partition split and each
original kernel's argument list.  All computation happens in libhfuse_gfx950.so
(hand-written HIP); this package is a thin ctypes mirror of its C-ABI."""
import os

from . import _lib
from ._lib import HfuseError, LIB_PATH  # noqa: F401
from .launcher import Config, Plan, launch_native  # noqa: F401

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "configs")


def default_config() -> Config:
    """The fusion list and kernel table shipped with the library."""
    return Config.from_files(os.path.join(CONFIG_DIR, "gfx950_fusion.yaml"),
                             os.path.join(CONFIG_DIR, "gfx950_kernels.yaml"))


def triples_config() -> Config:
    """The three-kernel fusions of the reference's lists over the same kernel table."""
    return Config.from_files(os.path.join(CONFIG_DIR, "gfx950_triples.yaml"),
                             os.path.join(CONFIG_DIR, "gfx950_kernels.yaml"))
