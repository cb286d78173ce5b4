"""Host-side Python view of libapnn_tc.so (the gfx950 wXaY GEMM / convolution library).

The directory name contains a hyphen, so import it by path:

    import importlib.util, sys
    spec = importlib.util.spec_from_file_location(
        "apnn_tc_amd", "<repo>/apnn-tc_amd/__init__.py",
        submodule_search_locations=["<repo>/apnn-tc_amd"])
    mod = importlib.util.module_from_spec(spec); sys.modules["apnn_tc_amd"] = mod
    spec.loader.exec_module(mod)

Python is only a convenience for tests and benchmarks; the product is the C ABI in
include/apnn_tc.h.  There is no CPU fallback: every call goes to the HIP library.
"""
from .binding import *  # noqa: F401,F403
from .binding import __all__ as _b_all
from .nn_binding import *  # noqa: F401,F403
from .nn_binding import __all__ as _n_all

__all__ = list(_b_all) + list(_n_all)
