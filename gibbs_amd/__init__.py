"""gibbs_amd: a small, whole LFM2 inference engine for one AMD MI355X.

    from gibbs_amd import Engine, generate
    engine = Engine("model_dir", dtype="bfloat16")
    out = generate(engine, [[5, 17, 42]], max_tokens=16, temperature=0.0)
"""
from .config import Lfm2Config, config_from_dict, register_architecture
from .engine import (ContinuousBatchScheduler, Engine, Entry, Generation, Generator, OutOfPages, StepError,
                     generate)
from .sampling import SamplingParams

__all__ = ["Engine", "Entry", "OutOfPages", "StepError", "Lfm2Config", "config_from_dict",
           "register_architecture", "ContinuousBatchScheduler", "Generator", "Generation", "generate",
           "SamplingParams"]
