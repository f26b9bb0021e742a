"""yalm_amd: a small generation library for the Llama / Mistral dense decoder on
MI355X (gfx950): typed configuration and registry, weights by name, layers put
together from parts, a paged cache with slots, one step function, a generation
loop with sampling, hand-written HIP kernels, and trace replay.

    from yalm_amd import Model, Engine, generate
    model = Model.from_folder("path/to/model", dtype=torch.bfloat16)
    engine = Engine(model, max_tokens=8192)
    new_tokens = generate(engine, [[1, 5, 17]], max_new_tokens=32, temperature=0.0)
"""
from . import parts  # noqa: F401  (registers the parts)
from .config import config_from_dict, config_from_folder, register_architecture
from .engine import Engine, Model, StepError
from .generate import GenerationStats, generate
from .parts import register_part
from .sampling import Sampler
from .weights import write_random_model

__all__ = ["Engine", "Model", "StepError", "GenerationStats", "generate", "Sampler", "config_from_dict",
           "config_from_folder", "register_architecture", "register_part", "write_random_model"]
