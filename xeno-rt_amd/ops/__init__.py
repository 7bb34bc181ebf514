"""The kernel library: hand-written HIP for gfx950, loaded from the in-tree shared library."""


def load_ops():
    """The HIP kernels, or an error: the engine has no other way to compute."""
    from .hip import HipOps
    return HipOps.instance()
