"""From a model folder (or a config and a weight source) to a runner: model, cache manager, step function.

The reference's wiring is ModelLoader.prepare / newBackend (ModelLoader.java:506-524, :658-759): read
config.json, open the weights, size the context and the KV pool, build the backend.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..cache.manager import CacheManager
from ..config import ModelConfig, entry_for, load_config
from ..parts.model import DecoderModel
from ..weights.safetensors_io import SafetensorsSource
from .step import ModelRunner

DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
          "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}") from None


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine runs its model on an AMD GPU through HIP kernels only")
    return torch.device("cuda", torch.cuda.current_device())


def build_model(config: ModelConfig, source, dtype, device, max_positions: int):
    """The model class comes from the registry entry of the config's model_type."""
    entry = entry_for(config.model_type)
    factory = entry.model_factory or DecoderModel
    model = factory(config, parse_dtype(dtype), device, max_positions)
    model.load(source)
    return model


def load_model(model_dir: str, dtype="bfloat16", device=None, max_positions: Optional[int] = None):
    config = load_config(model_dir)
    source = SafetensorsSource(model_dir)
    device = device or require_gpu()
    return build_model(config, source, dtype, device, max_positions or config.max_positions)


def build_runner(model, page_size: int = 16, pool_tokens: int = 0, max_requests: int = 4,
                 max_positions: Optional[int] = None, graphs: Optional[bool] = None,
                 prefix_share: bool = False) -> ModelRunner:
    """``pool_tokens`` positions of cache in pages of ``page_size``; 0 = room for every request at full length
    (cpu/CpuBackend.java:188-191: slots x (ceil(ctx / block) + 2) blocks by default). ``graphs``: replay
    captured decode steps (default: on for bfloat16 on the GPU). ``prefix_share``: requests whose tokens start
    alike share the pages of that start (backend.kv-prefix-share, jllm.properties:117-118); a model that cannot
    (a window, per-request state) runs without, and ``runner.cache.sharing_refused`` says why."""
    max_positions = max_positions or model.build.max_positions
    if pool_tokens <= 0:
        pool_tokens = max_requests * (-(-max_positions // page_size) + 2) * page_size
    cache = CacheManager(model.cache_plans(), page_size, pool_tokens, max_requests, dtype=model.dtype,
                         device=model.device, prefix_share=prefix_share)
    runner = ModelRunner(model, cache, max_positions)
    if graphs is None:
        graphs = model.dtype == torch.bfloat16 and model.device.type == "cuda"
    if graphs:
        from .graphs import DecodeGraphs
        runner.graphs = DecodeGraphs(runner, max_requests)
    return runner
