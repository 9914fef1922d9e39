"""gibbs_amd: a small, whole LFM2 inference engine for one AMD MI355X."""
from .config import Lfm2Config, config_from_dict, register_architecture
from .engine import Engine, Entry, OutOfPages, StepError

__all__ = ["Engine", "Entry", "OutOfPages", "StepError", "Lfm2Config", "config_from_dict", "register_architecture"]
