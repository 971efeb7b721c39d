"""Where tensors come from: a safetensors folder, or a seeded random generator.

Both answer ``names()`` -> {tensor name: (shape, dtype string)} and
``fetch(name)`` -> a CPU (or device) tensor, so the loader validates and binds
them the same way.
"""

from __future__ import annotations

import zlib
from pathlib import Path
from typing import Callable, Mapping

import torch
from safetensors import safe_open

_ST_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}


class SafetensorsSource:
    """All ``*.safetensors`` files of a folder, sorted by name
    (reference: src/tokamak/model/loader.py:67-69)."""

    def __init__(self, folder: str | Path) -> None:
        self.folder = Path(folder)
        self.files = sorted(self.folder.glob("*.safetensors"))
        if not self.files:
            raise FileNotFoundError(f"No *.safetensors files found under {self.folder}")
        self._where: dict[str, Path] = {}
        self._meta: dict[str, tuple[tuple[int, ...], torch.dtype]] = {}
        for file in self.files:
            with safe_open(file, framework="pt", device="cpu") as f:
                for name in f.keys():
                    sl = f.get_slice(name)
                    self._where[name] = file
                    self._meta[name] = (tuple(sl.get_shape()), _ST_DTYPES[sl.get_dtype()])

    def names(self) -> Mapping[str, tuple[tuple[int, ...], torch.dtype]]:
        return self._meta

    def fetch(self, name: str) -> torch.Tensor:
        with safe_open(self._where[name], framework="pt", device="cpu") as f:
            return f.get_tensor(name)


class RandomSource:
    """Seeded random tensors for a list of expected names.

    Every tensor has a generator of its own, seeded from (seed, crc32(name)),
    so values do not depend on the order tensors are asked for.  Values are
    drawn in float32 and stored in ``dtype``: matrices ~ N(0, matrix_std);
    vectors (norm weights) 1 + N(0, vector_jitter).
    """

    def __init__(
        self,
        expected: Mapping[str, "TensorSpec"],
        seed: int,
        *,
        matrix_std: float = 0.02,
        vector_jitter: float = 0.0,
        dtype: torch.dtype = torch.bfloat16,
        device: str | torch.device = "cpu",
        init: Callable[[str, "TensorSpec"], torch.Tensor | None] | None = None,
    ) -> None:
        self.expected = dict(expected)
        self.seed = int(seed)
        self.matrix_std = matrix_std
        self.vector_jitter = vector_jitter
        self.dtype = dtype
        self.device = torch.device(device)
        self.init = init

    def names(self) -> Mapping[str, tuple[tuple[int, ...], torch.dtype]]:
        return {n: (tuple(s.shape), self.dtype) for n, s in self.expected.items()}

    def fetch(self, name: str) -> torch.Tensor:
        spec = self.expected[name]
        if self.init is not None:
            custom = self.init(name, spec)
            if custom is not None:
                return custom.to(self.dtype)
        gen = torch.Generator(device=self.device)
        gen.manual_seed((self.seed * 1000003 + zlib.crc32(name.encode())) % (2**63))
        x = torch.randn(tuple(spec.shape), generator=gen, dtype=torch.float32, device=self.device)
        if spec.role == "vector":
            x = 1.0 + self.vector_jitter * x
        else:
            x = self.matrix_std * x
        return x.to(self.dtype)


from tokamak_amd.weights.spec import TensorSpec  # noqa: E402  (type used above)
