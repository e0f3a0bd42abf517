"""The checks that pin the oracle and the host-side logic, collected a second time under the `gpu` mark.

They need no GPU.  They are what makes "equal to the oracle" mean something, so they also run where the GPU
parity tests run: the same functions as in test_oracle_pins.py, test_golden_oracle.py and the host-only part of
test_capi_cpu.py, imported here so that `-m gpu` selects them too.
"""
import pytest

from test_capi_cpu import (capi, test_header_declares_the_index_level_boundary,  # noqa: F401
                           test_library_exports_every_declared_symbol, test_merge_search_results_matches_the_oracle,
                           test_merge_search_results_rejects_bad_arguments, test_product_never_imports_the_oracle,
                           test_scan_lds_plan_keeps_every_region_inside_the_allocation)
from test_golden_oracle import *  # noqa: F401,F403
from test_oracle_pins import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu
