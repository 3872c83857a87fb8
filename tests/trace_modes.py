"""The replay traces of the tests: the framework's own builders (`inferrs_amd.engine.trace`)."""
from inferrs_amd.engine.trace import (MODES, Trace, make_trace, mixed, portions, prefix_then_single,  # noqa: F401
                                      round_up, whole)
