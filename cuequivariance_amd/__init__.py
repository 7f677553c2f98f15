"""MI355X-native execution engine for cuEquivariance's segmented-polynomial operations.

``cuequivariance_amd.cue``  : descriptor side (irreps, Clebsch-Gordan, segmented tensor products).
``cuequivariance_amd.cuet`` : torch modules with the ``cuequivariance_torch`` API, running HIP kernels
                              through the C ABI of ``libcueq_amd.so``.
"""

__version__ = "0.1.0"

from . import cue  # noqa: F401


def __getattr__(name):
    # torch is imported only when the torch-facing layer is requested
    if name == "cuet":
        import importlib

        return importlib.import_module(".cuet", __name__)
    raise AttributeError(name)
