"""Imports the package directory `grab-anns_amd` (not a valid module name) as `grab_anns_amd`."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load():
    if "grab_anns_amd" in sys.modules:
        return sys.modules["grab_anns_amd"]
    path = os.path.join(ROOT, "grab-anns_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("grab_anns_amd", path,
                                                  submodule_search_locations=[os.path.dirname(path)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["grab_anns_amd"] = mod
    spec.loader.exec_module(mod)
    return mod
