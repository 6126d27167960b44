"""Launch-time keyword flags of the reference, accepted and ignored.

The reference passes compiler options as extra keyword arguments on the
kernel launch (`kernel[grid](..., enableHexKL=True, iterations=1)`); they are
the fields of `HexagonOptions` (qcom_hexagon_backend/backend/hexagon_options.py:16-120),
filtered out of the kernel arguments in `parse_options`
(qcom_hexagon_backend/backend/compiler.py:160-185). The kernels here are
precompiled, so the flags select nothing, but call sites written for the
reference keep working: a known flag is dropped, an unknown keyword is an
error exactly as a misspelt option would be there.
"""

OPTION_NAMES = frozenset((
    "allow_fp8e4nv", "allowed_dot_input_precisions", "arch_triple", "arch_features", "device_type",
    "vectorize", "vector_length", "num_threads", "data_layout", "num_warps", "num_stages", "num_ctas",
    "shared", "cluster_dims", "supported_fp8_dtypes", "sanitize_overflow", "debug", "name",
    "instrumentation_mode", "htp_kernel_gen", "target_artifact", "iterations",
    "fusion", "fusionAllowRecompute", "fusionDoMultiUse", "enableBufferization",
    "enableCollapseAddressSpace", "enableConvTiling", "enableDoubleBuffering", "convTileSizes",
    "enableConvertToHexagonmem", "enableHexagonmemCopyToDMA", "enableHexKL", "hexKLMode",
    "enableMultiThreading", "enableThreadedDispatch", "enableSCFThreading", "enableSplitReduction",
    "enableSplitReduceGeneric", "enableVectorization", "enableVTCMTiling", "scratch", "enableHVXInlining",
    "enableSCFLoopUnroll", "enableConversionToFp16", "enableSeedLayoutConversions", "tileSizes",
    "lowerConstantsInSeparateSharedObjects", "enableLWP", "disableLWPLoop", "LWPloopDepth", "deviceCleanup",
))


def split_options(kwargs):
    """Return (kernel_kwargs, option_kwargs); option_kwargs are reference flags."""
    kernel, opts = {}, {}
    for k, v in kwargs.items():
        (opts if k in OPTION_NAMES else kernel)[k] = v
    return kernel, opts
