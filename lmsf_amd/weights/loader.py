"""Loads a model's weights by tensor name and checks them against what its parts declare.

The reference reads each tensor where the layer is built (``vb.get(shape, name)``,
core/src/model_executor/layers/linear.rs:285-290; names in models/llama/llama.rs:185-189, :265-267,
:485-495) and fails on the first problem, partly by panic (llama.rs:506). Here every part declares
its checkpoint tensors first; the file set is compared with the declarations once, and a single
error lists every missing tensor, every unexpected tensor and every wrong shape.

Element types: a tensor declared "float" is cast to the run's type as the reference casts at load
(core/src/model_executor/models/model_factory.rs:124-139, core/src/common/config.rs:181-186): bfloat16 in
a bfloat16 run (float16 and float32 storage are converted), float32 in a float32 run. A tensor stored in
32 bits stays in 32 bits in a bfloat16 run where its declaration says so (``TensorDecl.keeps_float32``: the
norms' weights) or where the caller asks for it for all of them (``keep_float32``: the matrices' products
then run in float32 arithmetic, at twice the memory). A tensor declared "int" becomes int32.
"""
import warnings
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from ..parts.base import Part, TensorDecl
from .safetensors_io import SafetensorsError, SafetensorsFile, TensorEntry, list_weight_files


class WeightsError(ValueError):
    """The checkpoint does not fit the model. ``missing``, ``unexpected`` and ``wrong_shape`` hold
    the tensor names (wrong_shape: (name, expected, found))."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def collect_declarations(parts: Iterable[Part], shared: Optional[set] = None) -> Dict[str, TensorDecl]:
    """Every declared tensor by name; ``shared`` (a set, if given) takes the names that more than one part
    declares (tied weights)."""
    decls: Dict[str, TensorDecl] = {}
    for p in parts:
        for name, decl in p.checkpoint_tensors().items():
            if name in decls:
                if decls[name].shape != decl.shape:
                    raise ValueError("tensor %r is declared twice with shapes %s and %s"
                                     % (name, decls[name].shape, decl.shape))
                if shared is not None:
                    shared.add(name)
            decls[name] = decl
    return decls


def check_against_declarations(decls: Dict[str, TensorDecl], found: Dict[str, Tuple[int, ...]],
                               tolerated: Sequence[str] = (), where: str = "checkpoint") -> None:
    """Raise one WeightsError naming everything that does not fit; return if all fits."""
    missing = sorted(n for n in decls if n not in found)
    tolerated_set = set(tolerated)
    unexpected = sorted(n for n in found if n not in decls and n not in tolerated_set
                        and not any(n.endswith(suffix) for suffix in tolerated if suffix.startswith(".")))
    wrong = sorted((n, tuple(decls[n].shape), tuple(found[n])) for n in decls
                   if n in found and tuple(found[n]) != tuple(decls[n].shape))
    if not (missing or unexpected or wrong):
        return
    lines = ["%s does not fit the model:" % where]
    if missing:
        lines.append("  missing tensors (%d): %s" % (len(missing), ", ".join(missing)))
    if unexpected:
        lines.append("  unexpected tensors (%d): %s" % (len(unexpected), ", ".join(unexpected)))
    if wrong:
        lines.append("  wrong shapes (%d): %s" % (len(wrong), "; ".join(
            "%s expected %s found %s" % (n, list(e), list(f)) for n, e, f in wrong)))
    raise WeightsError("\n".join(lines), missing, unexpected, wrong)


def _convert(t: torch.Tensor, decl: TensorDecl, run_dtype: torch.dtype, keep_float32: bool = False) -> torch.Tensor:
    if decl.kind == "int":
        if t.dtype.is_floating_point or t.dtype == torch.bool:
            raise WeightsError("tensor declared as integer table is stored as %s" % t.dtype)
        return t.to(torch.int32)
    if not t.dtype.is_floating_point:
        raise WeightsError("tensor declared as float is stored as %s" % t.dtype)
    if run_dtype == torch.float32:
        return t.to(torch.float32)
    if t.dtype in (torch.float32, torch.float64) and (decl.keeps_float32 or keep_float32):
        return t.to(torch.float32)          # stored in 32 bits (or more) and meant to stay so
    return t.to(run_dtype)


def _return_freed_memory(device) -> None:
    """Source tensors are freed as soon as they are copied into their part's buffers, but torch keeps their
    blocks and would cut the next weights out of them, leaving holes that it can neither use for the cache's
    large tensors nor give back (12.9 GB of them after a 141 GB model). So what has been freed goes back to the
    device between parts, whenever it is more than 64 MB."""
    device = torch.device(device)
    if device.type != "cuda":
        return
    if torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device) > (64 << 20):
        torch.cuda.empty_cache()


def load_weights(parts: Sequence[Part], folder: str, device: torch.device, run_dtype: torch.dtype,
                 tolerated: Sequence[str] = (), keep_float32: bool = False) -> None:
    """Check the checkpoint in ``folder`` against the parts' declarations, then hand every part its
    tensors on ``device``. A name declared by two parts (tied weights) is loaded once and shared.
    ``keep_float32``: every tensor stored in 32 bits stays so in a bfloat16 run (see the module's text)."""
    parts = list(parts)
    shared: set = set()
    decls = collect_declarations(parts, shared)
    try:
        files = [SafetensorsFile(p) for p in list_weight_files(folder)]
    except SafetensorsError as e:
        raise WeightsError(str(e))
    try:
        entries: Dict[str, Tuple[SafetensorsFile, TensorEntry]] = {}
        for f in files:
            for name, e in f.entries.items():
                if name in entries:
                    raise WeightsError("tensor %r is in both %s and %s" % (name, entries[name][1].file, e.file))
                entries[name] = (f, e)
        check_against_declarations(decls, {n: e.shape for n, (_, e) in entries.items()}, tolerated,
                                   where="checkpoint %r" % folder)
        cache: Dict[str, torch.Tensor] = {}      # only what several parts share: the rest belongs to its part
        kept_wide: List[str] = []

        def fetch(name: str) -> torch.Tensor:
            if name not in decls:
                raise KeyError("part asked for tensor %r that it did not declare" % name)
            if name in cache:
                return cache[name]
            f, _ = entries[name]
            try:
                if torch.device(device).type == "cuda":
                    # from the mapped file to the device as stored, converted there: the bytes are passed over once
                    # on the host, and a 32-bit checkpoint is cast by the GPU
                    t = _convert(f.read(name, copy=False).to(device), decls[name], run_dtype, keep_float32)
                else:
                    t = _convert(f.read(name), decls[name], run_dtype, keep_float32)
            except WeightsError as e:
                raise WeightsError("%s: %s" % (name, e))
            if t.dtype == torch.float32 and run_dtype != torch.float32 and t.dim() >= 2:
                kept_wide.append(name)
            t = t.to(device)
            if name in shared:
                cache[name] = t
            return t

        for p in parts:
            p.load_weights(fetch)
            _return_freed_memory(device)
        if kept_wide:
            warnings.warn("%d matrices of %r are stored in 32 bits and stay so in this %s run (first: %s): their "
                          "products run without the matrix cores and they take twice the memory; store the "
                          "checkpoint in bfloat16 for speed" % (len(kept_wide), folder, run_dtype, kept_wide[0]))
    finally:
        for f in files:
            f.close()


def load_weights_from_generator(parts: Sequence[Part], make: Callable[[str, TensorDecl], torch.Tensor],
                                device=None) -> None:
    """Hand every part tensors made by ``make(name, declaration)`` (random weights on the device)."""
    parts = list(parts)
    shared: set = set()
    decls = collect_declarations(parts, shared)
    cache: Dict[str, torch.Tensor] = {}

    def fetch(name: str) -> torch.Tensor:
        if name not in decls:
            raise KeyError("part asked for tensor %r that it did not declare" % name)
        if name in cache:
            return cache[name]
        t = make(name, decls[name])
        if tuple(t.shape) != tuple(decls[name].shape):
            raise WeightsError("generated tensor %r has shape %s, declared %s"
                               % (name, list(t.shape), list(decls[name].shape)))
        if name in shared:
            cache[name] = t
        return t

    for p in parts:
        p.load_weights(fetch)
        if device is not None:
            _return_freed_memory(device)
