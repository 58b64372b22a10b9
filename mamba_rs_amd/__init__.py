"""MI355X-native Mamba inference hot path (HIP kernels behind a C ABI).

The compute lives in libmamba_hip.so (csrc/*.hip, built for gfx950); this
package is the thin host side: ctypes binding, operator wrappers and the
engine types that mirror the reference's GpuMambaBackbone surface.
"""
from ._lib import MambaHipError, load as load_library  # noqa: F401
from .config import MambaConfig, ScanMode, WeightDtype, PARALLEL_SCAN_THRESHOLD  # noqa: F401
from .weights import MambaWeights, MambaLayerWeights  # noqa: F401
from .backbone import GpuMambaBackbone, GpuMambaLM, SampleParams  # noqa: F401
from .mamba3 import Mamba3Config, Mamba3Weights, Mamba3LayerWeights, GpuMamba3Backbone  # noqa: F401

GpuMamba3LM = GpuMambaLM   # the same loop; the constructor picks the engine type (src/module/gpu_lm3.rs)
from . import formats  # noqa: F401
from .formats import load_hf, save_hf, parse_config_json, remap_m1_hf_key, HfMambaConfig, HfModel  # noqa: F401
