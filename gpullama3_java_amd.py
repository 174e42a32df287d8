"""Import alias: ``import gpullama3_java_amd`` loads the package in ``gpullama3.java_amd/``.

The package folder carries a dot in its name, which the import system reads as a
sub-module separator; this module loads that folder under an importable name and
puts the package in its own place in ``sys.modules``.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpullama3.java_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_pkg = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _pkg
_spec.loader.exec_module(_pkg)
