from .driver import HipDriver, LoadedKernel, get_driver, load_kernel  # noqa: F401
