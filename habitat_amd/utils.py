"""The helpers of the reference's `habitat.utils` that the prediction path uses
(analyzer/habitat/utils.py:46-63): unit conversions and the merge of positional
and keyword arguments by parameter name.  The command-line helpers of that
module belong to the profiling tools and are not part of this package."""
from habitat_amd.analysis.predictor import name_all_arguments  # noqa: F401
from habitat_amd.analysis.run_time import ms_to_ns  # noqa: F401


def ns_to_ms(ns):
    return ns / 1e6
