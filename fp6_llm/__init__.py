"""`import fp6_llm` for callers of usyd-fsalab/fp6_llm: the names that package exports (fp6_llm/__init__.py:1-23 of the
reference), served by the MI355X engine in fp6_llm_amd.  Nothing lives here; see fp6_llm_amd for the API."""
from fp6_llm_amd import (HeuristicFuntion_SplitK, Num_Wave, linear_forward_cuda, linear_forward_eXmY_cuda, weight_dequant_cpu,  # noqa: F401
                         weight_dequant_eXmY_cpu, weight_prepacking_cpu, weight_prepacking_eXmY_cpu)

__all__ = ["linear_forward_cuda", "weight_prepacking_cpu", "weight_dequant_cpu", "linear_forward_eXmY_cuda", "weight_prepacking_eXmY_cpu",
           "weight_dequant_eXmY_cpu", "Num_Wave", "HeuristicFuntion_SplitK"]
