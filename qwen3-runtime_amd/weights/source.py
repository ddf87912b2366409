"""Where tensors come from: a model folder's safetensors files, or a seed.

Both sources answer the same three questions: which names exist, what shape
and dtype a name has (without reading its data), and the tensor itself. A
folder is read through ``model.safetensors.index.json`` when present, else
through every ``*.safetensors`` file in it
(reference: qwen3_runtime/utils/loader.py:63-81); tensors are opened lazily,
one at a time, so that a large model never sits in host memory twice.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Iterable, Sequence

import torch

from ..parts.plan import TensorDecl

_ST_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}


class SafetensorsSource:
    def __init__(self, folder: str | Path):
        from safetensors import safe_open

        self.folder = Path(folder)
        index = self.folder / "model.safetensors.index.json"
        if index.exists():
            weight_map = json.loads(index.read_text()).get("weight_map") or {}
            files = sorted(set(weight_map.values()))
            if not files:
                raise FileNotFoundError(f"empty weight_map in {index}")
            paths = [self.folder / f for f in files]
        else:
            paths = sorted(self.folder.glob("*.safetensors"))
            if not paths:
                raise FileNotFoundError(f"no .safetensors files in {self.folder}")
        self._handles = []
        self._where: dict[str, int] = {}
        for path in paths:
            if not path.is_file():
                raise FileNotFoundError(f"{path} is named by the index but does not exist")
            handle = safe_open(str(path), framework="pt", device="cpu")
            self._handles.append(handle)
            for name in handle.keys():
                self._where[name] = len(self._handles) - 1

    def names(self) -> list[str]:
        return sorted(self._where)

    def has(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self._handles[self._where[name]].get_slice(name).get_shape())

    def dtype(self, name: str) -> torch.dtype:
        return _ST_DTYPES[self._handles[self._where[name]].get_slice(name).get_dtype()]

    def get(self, name: str, device: torch.device | str = "cpu") -> torch.Tensor:
        return self._handles[self._where[name]].get_tensor(name).to(device)


class RandomSource:
    """Seeded random tensors for a list of declarations.

    Each tensor is drawn from a generator seeded by (seed, tensor name), so its
    values do not depend on which other tensors exist or on the order they are
    asked for. ``"matrix"`` and ``"embedding"`` tensors are N(0, std);
    ``"norm"`` tensors are ``1 + N(0, norm_jitter)`` (all ones when the jitter
    is zero). Values are rounded to ``store_dtype``. Integer tables
    (``storage="int"``) are int32: zeros, or uniform in ``[0, n)`` for ``init="index:<n>"``.
    """

    def __init__(
        self,
        decls: Iterable[TensorDecl],
        seed: int,
        std: float = 0.02,
        norm_jitter: float = 0.1,
        store_dtype: torch.dtype = torch.bfloat16,
    ):
        self._decls = {d.file_name: d for d in decls}
        self.seed = int(seed)
        self.std = float(std)
        self.norm_jitter = float(norm_jitter)
        self.store_dtype = store_dtype

    def names(self) -> list[str]:
        return sorted(self._decls)

    def has(self, name: str) -> bool:
        return name in self._decls

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self._decls[name].shape)

    def dtype(self, name: str) -> torch.dtype:
        return torch.int32 if self._decls[name].storage == "int" else self.store_dtype

    def get(self, name: str, device: torch.device | str = "cpu") -> torch.Tensor:
        decl = self._decls[name]
        digest = hashlib.sha256(f"{self.seed}:{name}".encode()).digest()
        gen = torch.Generator(device=device)
        gen.manual_seed(int.from_bytes(digest[:8], "little") & (2**63 - 1))
        if decl.storage == "int":
            if decl.init.startswith("index:"):
                return torch.randint(0, int(decl.init[6:]), decl.shape, generator=gen, dtype=torch.int32,
                                     device=device)
            return torch.zeros(decl.shape, dtype=torch.int32, device=device)
        x = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=device)
        if decl.init == "norm":
            x = 1.0 + self.norm_jitter * x
        else:
            x = self.std * x
        return x.to(self.store_dtype)


def write_model_folder(
    folder: str | Path,
    config_json: dict,
    seed: int,
    *,
    std: float = 0.02,
    norm_jitter: float = 0.1,
    store_dtype: torch.dtype = torch.bfloat16,
    f32_names: Sequence[str] = (),
    device: torch.device | str = "cpu",
) -> Path:
    """Random-weights mode: write ``config.json`` and ``model.safetensors``.

    The architecture named by ``config_json`` decides which tensors exist.
    Names in ``f32_names`` are stored in float32 instead of ``store_dtype``.
    ``device``: where the values are drawn (a GPU draws a model of a real width in
    seconds where the host takes minutes; the values of a seed differ between devices).
    """
    from safetensors.torch import save_file

    from ..parts.model import DecoderModel
    from ..registry import architecture_for

    arch = architecture_for(config_json)
    model = DecoderModel(arch.make_plan(arch.read_config(config_json)))
    decls = model.tensor_decls()
    source = RandomSource(decls, seed, std=std, norm_jitter=norm_jitter, store_dtype=torch.float32)
    tensors = {}
    for decl in decls:
        t = source.get(decl.file_name, device)
        keep_f32 = decl.file_name in f32_names or decl.storage == "int"  # integers stay int32
        # round through the storage type so that every reader sees equal values
        tensors[decl.file_name] = (t if keep_f32 else t.to(store_dtype)).contiguous().cpu()
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config_json, indent=1))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
