"""Builds what a model folder needs to run steps: configuration, model, weights, cache, executor.

This is the common base of the engine (scheduler + sampler on top) and of trace replay (nothing
on top). Reference: Worker::from + Worker::init_cache (core/src/worker/model_worker.rs:34-126) and
the sizing of the cache from free device memory (:128-162).
"""
import warnings
from dataclasses import dataclass
from typing import Any, Optional, Sequence

import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..cache.storage import CacheStorage, plan_groups
from ..config.model_config import ArchConfig
from ..config.registry import Architecture, get_architecture, load_model_config
from ..models.decoder import DecoderModel
from ..parts.base import Runtime
from ..weights.loader import load_weights, load_weights_from_generator
from ..weights.random_init import random_tensor
from .executor import ModelExecutor

_DTYPES = {"float32": torch.float32, "float": torch.float32, "bfloat16": torch.bfloat16,
           "float16": torch.bfloat16, "half": torch.bfloat16}


def resolve_dtype(name: Optional[str], config: ArchConfig) -> torch.dtype:
    """--dtype overrides config.json's torch_dtype (core/src/common/config.rs:181-186). float16
    checkpoints run in bfloat16 (with a warning: three bits of every weight's mantissa go): the kernels
    have two element types, float32 and bfloat16."""
    key = name if name not in (None, "auto") else config.torch_dtype
    if key not in _DTYPES:
        raise ValueError("dtype %r is not supported (float32, bfloat16)" % (key,))
    if key in ("float16", "half"):
        warnings.warn("dtype %s runs as bfloat16 here: weights stored in float16 are rounded to bfloat16's 8 bits "
                      "of mantissa; use --dtype float32 to keep all of them" % key)
    return _DTYPES[key]


@dataclass
class EngineCore:
    arch: Architecture
    config: ArchConfig
    rt: Runtime
    model: DecoderModel
    storage: CacheStorage
    executor: ModelExecutor
    max_model_len: int
    block_size: int


def _default_ops():
    from ..ops import get_ops
    return get_ops()


def build_model(arch: Architecture, config: ArchConfig, rt: Runtime, model_dir: Optional[str],
                load_format: str = "auto", seed: int = 0, keep_float32_weights: bool = False) -> DecoderModel:
    model = DecoderModel(arch.build_spec(config), rt)
    if load_format == "random":
        std = 0.02
        store = torch.float32 if rt.dtype == torch.float32 else torch.bfloat16
        load_weights_from_generator(model.parts(),
                                    lambda name, decl: random_tensor(name, decl, seed, std, store, rt.device),
                                    device=rt.device)
    elif load_format == "auto":
        if model_dir is None:
            raise ValueError("a model folder is needed unless load_format is 'random'")
        load_weights(model.parts(), model_dir, rt.device, rt.dtype, tolerated=arch.tolerated_tensors,
                     keep_float32=keep_float32_weights)
    else:
        raise ValueError("load_format %r unknown (auto, random)" % load_format)
    return model


def profile_num_pages(model: DecoderModel, rt: Runtime, block_size: int, gpu_memory_utilization: float,
                      max_num_batched_tokens: int, max_num_seqs: int, max_model_len: int) -> Sequence[int]:
    """Pages per cache group from the device memory that is free after the weights are loaded:
    (total * utilization - used - room for one step's activations) / bytes per page
    (core/src/worker/model_worker.rs:146-154). Groups that keep every key share the budget in
    proportion to their page size in bytes; a window group gets what its window can ever hold."""
    groups, _ = plan_groups(model.cache_requirements(), block_size)
    if not groups:
        return []
    es = 4 if rt.dtype == torch.float32 else 2
    # what torch has freed but keeps (the loader's source tensors) goes back first, so that "used" is what is
    # really held: the weights, the HIP context and the libraries' own buffers
    torch.cuda.empty_cache()
    free, total = torch.cuda.mem_get_info(rt.device)
    spec = model.spec
    # (the embedding's table and the head's matrix apart: the first is gathered from, the second meets wanted rows only)
    ends = {t.data_ptr() for p in (model.embedding, model.head) for t in p.tensors()}
    mats = [t for p in model.parts() for t in p.tensors() if t.dim() == 2 and t.data_ptr() not in ends]
    widest = max((t.shape[0] for t in mats), default=spec.hidden_size)
    wes = max((t.element_size() for t in mats), default=es)       # matrices kept in 32 bits have 32-bit products
    # one step's activations (float32 stream twice, three buffers of the widest product), the logits of every
    # request three times over (the decode steps' shared buffer, the caller's copy, the sampler's scratch), and
    # the metadata buffers and the kernels' pool of the captured decode steps
    act = max_num_batched_tokens * (spec.hidden_size * 4 * 2 + widest * max(es, wes) * 3) \
        + max_num_seqs * spec.vocab_size * 4 * 3 + (512 << 20)
    return pages_for_budget(groups, int(total * gpu_memory_utilization) - (total - free) - act, es, block_size,
                            max_num_batched_tokens, max_num_seqs, max_model_len)


def pages_for_budget(groups, budget: int, elem_size: int, block_size: int, max_num_batched_tokens: int,
                     max_num_seqs: int, max_model_len: int) -> Sequence[int]:
    """Pages per cache group from ``budget`` bytes: a window group gets what its window can ever hold, the
    groups that keep every key share the rest, the same number of pages each (their block tables run in step)."""
    counts = [0] * len(groups)
    for gi, g in enumerate(groups):
        if g.spec.window is not None:
            per_seq = (g.spec.window + max_num_batched_tokens) // block_size + 2
            counts[gi] = per_seq * max_num_seqs
            budget -= counts[gi] * g.bytes_per_page(elem_size)
    full = [gi for gi, g in enumerate(groups) if g.spec.window is None]
    if full:
        per_page_all = sum(groups[gi].bytes_per_page(elem_size) for gi in full)
        n = max(0, budget // per_page_all)
        n = min(n, max_num_seqs * (-(-max_model_len // block_size)) + 1)   # more can never be used
        for gi in full:
            counts[gi] = int(n)
    return counts


def load_engine_core(model_dir: Optional[str], dtype: Optional[str] = None, block_size: int = 16,
                     max_model_len: Optional[int] = None, num_pages: Optional[int] = None,
                     gpu_memory_utilization: float = 0.9, max_num_seqs: int = 256,
                     max_num_batched_tokens: Optional[int] = None, device: str = "cuda:0",
                     ops: Any = None, load_format: str = "auto", seed: int = 0,
                     config: Optional[ArchConfig] = None, enforce_eager: bool = False,
                     use_program: bool = True, keep_float32_weights: bool = False) -> EngineCore:
    """``num_pages``: pages of every cache group (tests, replay); None sizes the pools from free memory.
    ``keep_float32_weights``: matrices stored in 32 bits stay so in a bfloat16 run instead of being cast."""
    if config is None:
        if model_dir is None:
            raise ValueError("need a model folder or a configuration")
        arch, config = load_model_config(model_dir)
    else:
        arch = get_architecture(config.architecture)
    derived = config.max_position_embeddings
    if max_model_len is None:
        max_model_len = derived
    elif max_model_len > derived:
        # core/src/common/config.rs:146-153
        raise ValueError("max_model_len %d is greater than the model's context length %d (config.json)"
                         % (max_model_len, derived))
    if not (0 < gpu_memory_utilization <= 1.0):
        raise ValueError("gpu_memory_utilization must be in (0, 1], got %r" % gpu_memory_utilization)  # config.rs:245-250
    if block_size <= 0:
        raise ValueError("block_size must be > 0")
    run_dtype = resolve_dtype(dtype, config)
    dev = torch.device(device)
    if ops is None:
        ops = _default_ops()
    rt = Runtime(ops=ops, device=dev, dtype=run_dtype, max_positions=max_model_len)
    model = build_model(arch, config, rt, model_dir, load_format, seed, keep_float32_weights)
    groups, _ = plan_groups(model.cache_requirements(), block_size)
    if max_num_batched_tokens is None:
        max_num_batched_tokens = max(max_model_len, 2048)   # config.rs:301-307
    if num_pages is None:
        counts = profile_num_pages(model, rt, block_size, gpu_memory_utilization, max_num_batched_tokens,
                                   max_num_seqs, max_model_len)
        if any(c * block_size < max_model_len for c, g in zip(counts, groups) if g.spec.window is None):
            # core/src/worker/model_worker.rs:115-118
            raise RuntimeError("the cache has room for %d tokens, fewer than max_model_len %d; raise "
                               "gpu_memory_utilization or lower max_model_len"
                               % (min(counts) * block_size, max_model_len))
    else:
        counts = [int(num_pages)] * len(groups)
    storage = CacheStorage(model, rt, block_size, counts, num_state_slots=max_num_seqs)
    # (a step never holds more tokens than the pools that keep every key have room for: the program's workspace is
    # sized for that many at most)
    room = [c * block_size for c, g in zip(counts, groups) if g.spec.window is None]
    executor = ModelExecutor(model, storage, rt, max_model_len, use_graphs=not enforce_eager,
                             use_program=use_program, max_step_tokens=min([max_num_batched_tokens] + room),
                             max_step_seqs=max_num_seqs)
    return EngineCore(arch, config, rt, model, storage, executor, max_model_len, block_size)
