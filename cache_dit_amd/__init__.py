"""cache_dit_amd: MI355X (gfx950) native FP8 quantized-linear path behind
cache-dit's `quantize()` / `enable_cache(..., quantize_config=...)` API.

    import cache_dit_amd as cache_dit
    cache_dit.quantize(transformer, cache_dit.QuantizeConfig(quant_type="float8_per_row"))

Built quant types: `float8_per_row` (w8a8, dynamic per-token activation scales),
`float8_per_tensor` (w8a8, one dynamic scale per tensor; also the policy's fallback
pass) and `float8_weight_only` (w8a16). The kernels live in lib/libcdit_hip.so
(C ABI: include/cdit_hip.h); there is no CPU or eager fallback.
"""
from .quantization import QuantizeBackend
from .quantization import QuantizeConfig
from .quantization import load
from .quantization import quantize
from .quantization import remove_quantization_stats
from .caching import enable_cache
from .caching import load_quantize_config
from .nn import Fp8DynamicLinear
from .nn import Fp8DynamicLinearPerTensor
from .nn import Fp8WeightOnlyLinear
from .nn import fuse_gelu_tanh_
from .nn import share_activation_quant_
from .nn import group_sibling_linears_
from .nn import linear_batch
from .nn import linear_on_cat
from .nn import precompute_stage
from .patch_functors import StagePatchFunctor
from .patch_functors import apply_stage_patch
from .patch_functors import remove_stage_patch
from .ops import ln_modulate_quant
from .utils import check_quantized

__version__ = "0.1.0"

__all__ = [
    "QuantizeBackend",
    "QuantizeConfig",
    "quantize",
    "load",
    "remove_quantization_stats",
    "enable_cache",
    "load_quantize_config",
    "check_quantized",
    "Fp8DynamicLinear",
    "Fp8DynamicLinearPerTensor",
    "Fp8WeightOnlyLinear",
    "fuse_gelu_tanh_",
    "share_activation_quant_",
    "group_sibling_linears_",
    "linear_batch",
    "linear_on_cat",
    "precompute_stage",
    "StagePatchFunctor",
    "apply_stage_patch",
    "remove_stage_patch",
    "ln_modulate_quant",
]
