"""Host-side Python harness around the sessd3d C-ABI library (tests, benchmark, examples)."""
