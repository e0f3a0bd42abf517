"""MI355X-native IVFPQ / Flat search path behind the AscendIndexIVFPQ / AscendIndexFlat interface."""
from . import ascendfaiss  # noqa: F401
from .ascendfaiss import (METRIC_INNER_PRODUCT, METRIC_L2, AscendIndexFlat, AscendIndexFlatL2,  # noqa: F401
                          AscendIndexInt8Flat, AscendIndexIVFPQ, AscendIndexIVFPQConfig, IndexSdkError,
                          merge_search_results)
