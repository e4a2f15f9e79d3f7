"""flux_amd — MI355X (gfx950) implementation of Flux's single-GPU MoE hot path.

`flux_amd.capi` binds the C-ABI of libfluxmi_kernels.so; the classes and functions re-exported below
come from the C++ torch extension `flux_ths_pybind` and carry the names and signatures of
bytedance/flux's Python surface (python/flux/cpp_mod.py:97-180) for this path.
"""
__version__ = "0.1.0"

from . import capi  # noqa: F401


def _load_ths():
    import importlib.util
    import os

    import torch  # noqa: F401  (libtorch and the HIP runtime must be loaded first)

    from .build import ths_ext_path

    path = ths_ext_path()
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python -m flux_amd.build`")
    capi.load()
    spec = importlib.util.spec_from_file_location("flux_ths_pybind", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_THS_NAMES = (
    "MoeArguments", "DistEnvTPWithEP", "GemmGroupedV3AGScatter", "GemmGroupedV3GatherRS", "GemmGroupedV3",
    "Quantization", "BlockScaleGemm", "calc_scatter_index", "topk_scatter_reduce", "bitwise_check", "init_flux_shm",
    "moe_route_sort", "topk_weighted_gather_reduce", "uniform_initialize", "load_tuning_record",
    "ProfilingContext", "TuningRecord", "load_tuning_text",
)
_ths = None


def __getattr__(name):
    global _ths
    if name in _THS_NAMES or name == "flux_ths_pybind":
        if _ths is None:
            _ths = _load_ths()
        return _ths if name == "flux_ths_pybind" else getattr(_ths, name)
    raise AttributeError(f"module 'flux_amd' has no attribute {name!r}")
