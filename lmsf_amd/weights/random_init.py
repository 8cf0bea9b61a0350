"""Random-weights mode: fills a model's declared tensors from a seed.

The reference has no such mode (candle ``Init`` hints exist only as call arguments,
tops/src/rms_norm.rs:42-46). Values are drawn per tensor from a generator seeded by
(seed, tensor name), so they do not depend on the order in which tensors are made:
matrices and biases N(0, std), norm weights 1.
"""
import hashlib
import json
import os
from typing import Dict, Optional

import torch

from ..config.model_config import ArchConfig
from ..config.registry import Architecture, get_architecture
from ..parts.base import Runtime, TensorDecl
from .loader import collect_declarations
from .safetensors_io import write_safetensors

_STORAGE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16,
            "half": torch.float16, "float": torch.float32}


def tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, decl: TensorDecl, seed: int, std: float, dtype: torch.dtype,
                  device: torch.device) -> torch.Tensor:
    """The tensor ``name`` of the random model ``seed``. Values are made in float32 on ``device``
    and rounded to ``dtype``; CPU and GPU generators differ, a model is tied to where it was made."""
    if decl.kind == "int":
        return torch.zeros(decl.shape, dtype=torch.int32, device=device)
    if decl.init == "ones":
        return torch.ones(decl.shape, dtype=dtype, device=device)
    if decl.init == "zeros":
        return torch.zeros(decl.shape, dtype=dtype, device=device)
    if decl.init != "normal":
        raise ValueError("tensor %r: unknown init %r" % (name, decl.init))
    gen = torch.Generator(device=device)
    gen.manual_seed(tensor_seed(seed, name))
    t = torch.empty(decl.shape, dtype=torch.float32, device=device)
    t.normal_(0.0, std, generator=gen)
    return t.to(dtype)


def declared_tensors(arch: Architecture, config: ArchConfig) -> Dict[str, TensorDecl]:
    """Names and shapes of the checkpoint tensors of ``config``'s model, without building weights."""
    from ..models.decoder import DecoderModel  # local import: models import parts, parts import nothing of weights

    rt = Runtime(ops=None, device=torch.device("cpu"), dtype=torch.float32,
                 max_positions=config.max_position_embeddings)
    model = DecoderModel(arch.build_spec(config), rt)
    return collect_declarations(model.parts())


def write_random_model(folder: str, config: ArchConfig, seed: int = 0, std: float = 0.02,
                       dtype: Optional[str] = None) -> str:
    """Write ``folder``/config.json and ``folder``/model.safetensors for ``config`` with random
    weights of ``seed``. ``dtype`` (default: the configuration's torch_dtype) is the storage type."""
    arch = get_architecture(config.architecture)
    dtype_name = dtype or config.torch_dtype
    if dtype_name not in _STORAGE:
        raise ValueError("unknown storage dtype %r" % dtype_name)
    os.makedirs(folder, exist_ok=True)
    cfg_dict = config.to_dict()
    cfg_dict["torch_dtype"] = dtype_name
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg_dict, f, indent=2)
    decls = declared_tensors(arch, config)
    cpu = torch.device("cpu")
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      ((name, random_tensor(name, decl, seed, std, _STORAGE[dtype_name], cpu))
                       for name, decl in sorted(decls.items())),
                      metadata={"format": "pt", "seed": str(seed)})
    return folder
