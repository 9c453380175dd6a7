"""The architectures that come with the engine: every module in this folder registers its architecture when it is
imported, and importing this package imports them all. Adding an architecture is adding a file here (or anywhere
else, named to the engine as a plugin); no other file lists their names."""
import importlib
import pkgutil

for _module in pkgutil.iter_modules(__path__):
    importlib.import_module(f"{__name__}.{_module.name}")
