"""Imports the hyphen-named package directory apnn-tc_amd as module `apnn_tc_amd`."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load():
    if "apnn_tc_amd" in sys.modules:
        return sys.modules["apnn_tc_amd"]
    d = os.path.join(ROOT, "apnn-tc_amd")
    spec = importlib.util.spec_from_file_location("apnn_tc_amd", os.path.join(d, "__init__.py"),
                                                  submodule_search_locations=[d])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["apnn_tc_amd"] = mod
    spec.loader.exec_module(mod)
    return mod
