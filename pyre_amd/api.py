"""The Python entry points, in the reference's manner: ``load_model`` returns the
thing that generates and its configuration (`pyre/loader.py:33-79`), ``Scheduler``
takes requests and runs them (`pyre/scheduler.py:27-44,105-114`)."""

from __future__ import annotations

from pathlib import Path

import torch

from pyre_amd.config import PRESETS, EngineConfig, preset
from pyre_amd.engine.context import TORCH_DTYPES
from pyre_amd.engine.engine import Engine
from pyre_amd.engine.scheduler import Scheduler as _Scheduler
from pyre_amd.sampling.sampler import Sampler
from pyre_amd.weights import model_tensor_specs, random_state


def _dtype_name(dtype) -> str:
    if isinstance(dtype, torch.dtype):
        return {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    return dtype


def load_model(model_id_or_path: str, device: str = "cuda", dtype="bfloat16", random_seed: int | None = None,
               std: float = 0.02, gain_std: float = 0.0, num_blocks: int | None = None, **engine_options):
    """Returns ``(engine, config)``.

    ``model_id_or_path`` is a folder with ``config.json`` and ``*.safetensors``, or,
    together with ``random_seed``, the name of a preset shape whose weights are then
    drawn on the device. ``num_blocks`` is the reference's name for the number of
    cache pages (`pyre/scheduler.py:28`). Other keywords are fields of
    :class:`~pyre_amd.config.EngineConfig`.
    """
    if device == "cuda":
        device = "cuda:0"
    if num_blocks is not None:
        engine_options["num_pages"] = num_blocks
    ec = EngineConfig(dtype=_dtype_name(dtype), device=device, **engine_options)
    if Path(model_id_or_path).is_dir():
        engine = Engine.from_folder(model_id_or_path, ec)
    elif model_id_or_path in PRESETS:
        if random_seed is None:
            raise ValueError(f"{model_id_or_path!r} is a preset shape: pass random_seed to draw its weights")
        config = preset(model_id_or_path)
        state = random_state(model_tensor_specs(config), random_seed, std, gain_std,
                             TORCH_DTYPES[ec.dtype], device=device)
        engine = Engine.from_state(config, state, ec)
    else:
        raise FileNotFoundError(f"{model_id_or_path!r} is neither a model folder nor a preset "
                                f"({', '.join(sorted(PRESETS))}); nothing is downloaded")
    return engine, engine.config


class Scheduler(_Scheduler):
    """``Scheduler(engine, max_batch=...)``; ``add_request(prompt_ids, max_new_tokens,
    eos_id, temperature, seed) -> seq_id``; ``run() -> {seq_id: tokens}``."""

    def __init__(self, engine: Engine, max_batch: int | None = None, max_num_batched_tokens: int | None = None,
                 prefill_chunk: int | None = None):
        sampler = Sampler(engine.device, engine.engine_config.max_num_seqs)
        super().__init__(engine, max_batch, max_num_batched_tokens, prefill_chunk, sampler)


def generate(engine: Engine, prompts: list[list[int]], max_new_tokens: int = 16, temperature: float = 0.0,
             eos_id: int | None = None, seed: int = 0, **scheduler_options) -> list[list[int]]:
    """Generated tokens for each prompt, in the order given."""
    sched = Scheduler(engine, **scheduler_options)
    ids = [sched.add_request(p, max_new_tokens, eos_id, temperature, seed) for p in prompts]
    out = sched.run()
    return [out[i] for i in ids]


def generate_greedy(engine: Engine, input_ids: list[int], max_new_tokens: int, eos_id: int | None = None) -> list[int]:
    """Prompt followed by its greedy continuation (`pyre/model.py:203-215,344-362`)."""
    return list(input_ids) + generate(engine, [list(input_ids)], max_new_tokens, 0.0, eos_id)[0]
