"""hf_cpu_amd: a small, whole inference engine for one GPU (gfx950).

``load_engine(model_dir, dtype=...)`` reads a model folder (config.json +
model.safetensors) and returns an Engine whose ``step`` runs batches of prompt
portions and decoded tokens from a paged cache; ``session.Session.generate`` and the
command line (``cli``) sit on top of it. Configuration in ``config``, tensors in
``weights``, layer parts in ``parts``, the cache's books and memory in ``cache``, the step
function and the scheduler in ``engine``, sampling in ``sampling``, the HIP sources in
``csrc`` and their Python face in ``kernels``.
"""
from . import parts, models           # noqa: F401  (registration of parts and architectures)
from .config import Qwen2Config, config_from_dict, read_config
from .model import Model
from .plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from .registry import register_architecture, register_part
from .status import EngineError
from .weights import write_random_model

__all__ = ["EngineError", "LayerPlan", "Model", "ModelPlan", "PartSpec", "Qwen2Config", "ScheduleEntry",
           "config_from_dict", "load_engine", "read_config", "register_architecture", "register_part",
           "write_random_model"]


def load_engine(model_dir, dtype="bfloat16", device="cuda:0", **engine_args):
    """The engine for the model in ``model_dir``. ``engine_args`` go to Engine
    (page_tokens, n_pages or max_tokens, max_seqs, max_context)."""
    from .engine import Engine
    from .kernels import Ops
    from .model import compute_dtype
    ops = Ops(compute_dtype(dtype), device)
    return Engine(Model.from_dir(model_dir, dtype, ops), ops, **engine_args)
