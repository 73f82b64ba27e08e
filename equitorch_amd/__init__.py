"""MI355X-native sparse Clebsch-Gordan tensor products behind the Equitorch Python API."""
from . import constants, irreps, structs, utils  # noqa: F401

__all__ = ["constants", "irreps", "structs", "utils", "nn", "ops", "transforms"]


def __getattr__(name):
    # nn / ops need the HIP library; import them lazily so table construction works without it
    if name in ("nn", "ops", "transforms"):
        import importlib
        return importlib.import_module(f"{__name__}.{name}")
    raise AttributeError(name)
