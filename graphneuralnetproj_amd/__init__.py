"""MI355X-native Tiled-CSL SpMM: Python mirror of the C ABI in include/SpMM_API.h."""
from .spmm_api import (  # noqa: F401
    GenSparseMatrixBinFile,
    InitSparseMatrixA_API,
    SpMM_PlanLaunch,
    SpMM_SplitK_API,
    SpMM_SplitK_API_Planned,
    SpMM_SplitK_API_RowMajor,
    SpMM_SplitK_API_Strided,
    SPMM_FLAG_RELU,
    SPMM_FLAG_SEPARATE_REDUCTION,
    SpMM_SuggestSplitK,
    SpMMError,
    build_library,
    library_path,
    load_library,
    synth_activations,
    synth_weights,
)
