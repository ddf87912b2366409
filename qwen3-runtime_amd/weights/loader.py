"""Load a model's tensors by name, with one error for everything that is wrong.

The model's parts declare the tensors they read (name, shape). Before any data
is read the declarations are checked against the source: names the source
lacks, tensors whose shape differs, tensors stored in a type their part cannot
take (an integer tensor where a matrix is read, a floating one where an integer
table is) and tensors the source holds that no part reads are gathered into a
single ``WeightError``. The reference stops at the
first missing key and ignores extra tensors silently
(qwen3_runtime/utils/loader.py:33-54).

Placement: a tensor keeps the type it is stored in when that is bfloat16 or
float32 and the engine runs in bfloat16 (a float32 tensor stays float32);
float16 becomes bfloat16. An engine in float32 holds everything in float32.
Weights of norms are always held in float32; integer tables are held as int32. Fused matrices (q|k|v, gate|up)
are concatenated on the device, row blocks in the given order
(reference: qwen3_runtime/utils/loader.py:42-53).
"""

from __future__ import annotations

from typing import Sequence

import torch

from ..parts.plan import TensorDecl


FLOAT_STORAGE = (torch.bfloat16, torch.float32, torch.float16)
INT_STORAGE = (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8)


class WeightError(RuntimeError):
    def __init__(self, missing, wrong_shape, unexpected, where="", wrong_dtype=()):
        self.missing = list(missing)
        self.wrong_shape = list(wrong_shape)
        self.unexpected = list(unexpected)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"model weights do not match the architecture{where}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong types ({len(self.wrong_dtype)}): " + "; ".join(
                f"{n} is stored as {got}, expected {want}" for n, got, want in self.wrong_dtype))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        super().__init__("\n".join(lines))


def check_source(source, decls: Sequence[TensorDecl], ignorable: Sequence[str] = (), where: str = "") -> None:
    wanted = {d.file_name: tuple(d.shape) for d in decls}
    missing = [n for n in wanted if not source.has(n)]
    wrong = [
        (n, source.shape(n), shape)
        for n, shape in wanted.items()
        if source.has(n) and tuple(source.shape(n)) != shape
    ]
    wrong_dtype = []
    for d in decls:
        if not source.has(d.file_name):
            continue
        stored = source.dtype(d.file_name)
        allowed = INT_STORAGE if d.storage == "int" else FLOAT_STORAGE
        if stored not in allowed:
            wrong_dtype.append((d.file_name, str(stored).replace("torch.", ""),
                                "an integer type" if d.storage == "int" else "bfloat16, float32 or float16"))
    unexpected = [n for n in source.names() if n not in wanted and n not in ignorable]
    if missing or wrong or wrong_dtype or unexpected:
        raise WeightError(missing, wrong, unexpected, where, wrong_dtype)


class WeightLoader:
    """Hands device tensors to parts; equal requests share one tensor (tied head)."""

    def __init__(self, source, device: torch.device | str, dtype: torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, got {dtype}")
        self.source = source
        self.device = torch.device(device)
        self.dtype = dtype
        self._cache: dict[tuple, torch.Tensor] = {}
        self.num_bytes = 0

    def _placed_dtype(self, stored: torch.dtype) -> torch.dtype:
        if self.dtype == torch.float32:
            return torch.float32
        if stored == torch.float32:
            return torch.float32
        return torch.bfloat16

    def _remember(self, key, make):
        if key not in self._cache:
            t = make().contiguous()
            self._cache[key] = t
            self.num_bytes += t.numel() * t.element_size()
        return self._cache[key]

    def matrix(self, file_name: str) -> torch.Tensor:
        def make():
            t = self.source.get(file_name, self.device)
            return t.to(self._placed_dtype(t.dtype))

        return self._remember(("matrix", file_name), make)

    def fused(self, file_names: Sequence[str], dim: int = 0) -> torch.Tensor:
        def make():
            parts = [self.source.get(n, self.device) for n in file_names]
            target = self._placed_dtype(
                torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
            )
            return torch.cat([p.to(target) for p in parts], dim=dim)

        return self._remember(("fused", tuple(file_names), dim), make)

    def vector_f32(self, file_name: str) -> torch.Tensor:
        return self._remember(
            ("f32", file_name), lambda: self.source.get(file_name, self.device).to(torch.float32)
        )

    def table_i32(self, file_name: str) -> torch.Tensor:
        """An integer table (declared with ``storage="int"``), held as int32 in every mode."""
        return self._remember(
            ("i32", file_name), lambda: self.source.get(file_name, self.device).to(torch.int32)
        )

    def constant(self, tensor: torch.Tensor) -> torch.Tensor:
        """A tensor the part computed itself (a table of constants): placed as it is."""
        return tensor.to(self.device).contiguous()


def load_model(model, source, device, dtype, where: str = "") -> WeightLoader:
    """Check ``source`` against ``model``'s declarations, then load every part."""
    check_source(source, model.tensor_decls(), model.plan.ignorable, where)
    loader = WeightLoader(source, device, dtype)
    model.load(loader)
    return loader
