"""Safetensors-backed tensor store with the shard arithmetic the quantized loaders need.

Mirrors the part of server/text_generation_server/utils/weights.py that the GPTQ/AWQ
loader touches: the `WeightsLoader` protocol (:13-73), `DefaultWeightsLoader` for layers
left unquantized (:99-136) and `Weights` (:139-414: name routing with prefix and aliases,
`get_tensor`, `get_sharded`, `get_partial_sharded`, `get_packed_sharded`, `use_loader`).

Packed int32 tensors are never cast (they are eight 4-bit values in disguise); floating
tensors are cast to the model dtype.  A process group is anything with `rank()` and
`size()`; `SingleGroup` is the one-GPU case.
"""

from __future__ import annotations

from contextlib import contextmanager
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

# dtypes that carry packed or integer payloads and must survive loading untouched
# (utils/weights.py:219-229).
_KEEP_DTYPES = (torch.int8, torch.int16, torch.int32, torch.int64)


@dataclass(frozen=True)
class SingleGroup:
    """rank 0 of 1."""

    def rank(self) -> int:
        return 0

    def size(self) -> int:
        return 1


def split_blocks(total: int, blocks: Union[int, Sequence[int]]) -> List[int]:
    """Sizes of the tensors packed side by side in a dimension of length `total`.

    An int asks for that many equal blocks; a list gives proportions, e.g. [2, 1, 1] of
    1024 is [512, 256, 256] (utils/weights.py:417-442).
    """
    if isinstance(blocks, int):
        if blocks <= 0 or total % blocks:
            raise AssertionError(f"Prepacked is not divisible by {blocks}")
        return [total // blocks] * blocks
    parts = sum(blocks)
    if parts <= 0 or total % parts:
        raise AssertionError(f"Cannot split {total} in proportional blocks: {list(blocks)}")
    unit = total // parts
    return [unit * b for b in blocks]


class WeightsLoader:
    """Interprets raw checkpoint tensors for one quantization format."""

    def get_weights(self, weights: "Weights", prefix: str):
        raise NotImplementedError

    def get_weights_col_packed(self, weights: "Weights", prefix: str, block_sizes):
        raise NotImplementedError

    def get_weights_col(self, weights: "Weights", prefix: str):
        return weights.get_multi_weights_col([prefix], 0)

    def get_multi_weights_col(self, weights: "Weights", prefixes: List[str], dim: int):
        raise NotImplementedError

    def get_weights_row(self, weights: "Weights", prefix: str):
        raise NotImplementedError


@dataclass
class UnquantizedWeight:
    """A dense weight.  Dense linears are outside the int4 path: the tensor is only
    carried so that `modules_to_not_convert` layers load; the caller builds the layer."""

    weight: torch.Tensor

    def get_linear(self, bias):
        raise NotImplementedError(
            "dense linear layers are not part of this package; use the weight tensor "
            "with the serving stack's own linear"
        )


class DefaultWeightsLoader(WeightsLoader):
    """Dense [out, in] tensors: column-parallel splits dim 0, row-parallel dim 1."""

    def __init__(self, weight_class=UnquantizedWeight):
        self.weight_class = weight_class

    def get_weights(self, weights, prefix):
        return weights.get_tensor(f"{prefix}.weight")

    def get_weights_col_packed(self, weights, prefix, block_sizes):
        return self.weight_class(
            weights.get_packed_sharded(f"{prefix}.weight", dim=0, block_sizes=block_sizes)
        )

    def get_multi_weights_col(self, weights, prefixes, dim):
        parts = [weights.get_sharded(f"{p}.weight", dim=0) for p in prefixes]
        return self.weight_class(torch.cat(parts, dim=dim))

    def get_weights_row(self, weights, prefix):
        return self.weight_class(weights.get_sharded(f"{prefix}.weight", dim=1))


class Weights:
    """Named tensors spread over safetensors files, sliced lazily per shard."""

    def __init__(
        self,
        filenames: Sequence[Union[str, Path]],
        device,
        dtype,
        process_group=None,
        weights_loader: Optional[WeightsLoader] = None,
        aliases: Optional[Dict[str, List[str]]] = None,
        prefix: Optional[str] = None,
    ):
        self.device = device
        self.dtype = dtype
        self.process_group = process_group if process_group is not None else SingleGroup()
        self.weights_loader = weights_loader if weights_loader is not None else DefaultWeightsLoader()
        self.aliases = aliases or {}
        self.prefix = prefix
        self._handles: Dict[str, object] = {}
        self.routing: Dict[str, str] = {}
        for filename in filenames:
            for key in self._open(str(filename)).keys():
                if key in self.routing:
                    raise RuntimeError(
                        f"Key {key} was found in multiple files: {filename} and {self.routing[key]}"
                    )
                self.routing[key] = str(filename)

    # -- storage ----------------------------------------------------------------------

    def _open(self, filename: str):
        handle = self._handles.get(filename)
        if handle is None:
            from safetensors import safe_open

            handle = safe_open(filename, framework="pytorch")
            self._handles[filename] = handle
        return handle

    def get_filename(self, tensor_name: str) -> Tuple[str, str]:
        """(file, stored name): the bare name, then `prefix.name`, each with its aliases."""
        candidates = [tensor_name]
        if self.prefix is not None:
            candidates.append(f"{self.prefix}.{tensor_name}")
        for name in candidates:
            for stored in [name, *self.aliases.get(name, [])]:
                filename = self.routing.get(stored)
                if filename is not None:
                    return filename, stored
        raise RuntimeError(f"weight {tensor_name} does not exist")

    def has_tensor(self, tensor_name: str) -> bool:
        try:
            self.get_filename(tensor_name)
        except RuntimeError:
            return False
        return True

    def _get_slice(self, tensor_name: str):
        filename, stored = self.get_filename(tensor_name)
        return self._open(filename).get_slice(stored)

    def get_shape(self, tensor_name: str):
        return tuple(self._get_slice(tensor_name).get_shape())

    def _place(self, tensor: torch.Tensor, to_device: bool = True, to_dtype: bool = True):
        if to_dtype and tensor.dtype not in _KEEP_DTYPES and tensor.dtype != self.dtype:
            tensor = tensor.to(dtype=self.dtype)
        if to_device:
            tensor = tensor.to(device=self.device)
        return tensor

    # -- whole and sharded reads ------------------------------------------------------

    def get_tensor(self, tensor_name: str, to_device: bool = True, to_dtype: bool = True):
        filename, stored = self.get_filename(tensor_name)
        return self._place(self._open(filename).get_tensor(stored), to_device, to_dtype)

    def get_partial_sharded(self, tensor_name: str, dim: int, to_device=True, to_dtype=True):
        """This rank's ceil(size / world) slab of `dim`; the last rank may get less."""
        slice_ = self._get_slice(tensor_name)
        world, rank = self.process_group.size(), self.process_group.rank()
        size = slice_.get_shape()[dim]
        block = (size + world - 1) // world
        return self._place(_cut(slice_, dim, rank * block, (rank + 1) * block), to_device, to_dtype)

    def get_sharded(self, tensor_name: str, dim: int, to_device=True, to_dtype=True):
        size = self._get_slice(tensor_name).get_shape()[dim]
        world = self.process_group.size()
        assert size % world == 0, (
            f"The choosen size {size} is not compatible with sharding on {world} shards"
        )
        return self.get_partial_sharded(tensor_name, dim, to_device=to_device, to_dtype=to_dtype)

    def get_packed_sharded(self, tensor_name: str, dim: int, block_sizes, to_dtype=True):
        """Shard a tensor that packs several projections (q|k|v, gate|up) along `dim`, so
        that every rank receives its share of each of them (utils/weights.py:281-345)."""
        slice_ = self._get_slice(tensor_name)
        world, rank = self.process_group.size(), self.process_group.rank()
        pieces, offset = [], 0
        for block in split_blocks(slice_.get_shape()[dim], block_sizes):
            assert block % world == 0, f"Prepacked tensor cannot be sharded across {world} shards"
            share = block // world
            pieces.append(_cut(slice_, dim, offset + rank * share, offset + (rank + 1) * share))
            offset += block
        tensor = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=dim)
        return self._place(tensor, True, to_dtype)

    def get_tensor_shard(self, var: torch.Tensor, dim: int):
        world, rank = self.process_group.size(), self.process_group.rank()
        block = var.size()[dim] // world
        return _cut(var, dim, rank * block, (rank + 1) * block).to(dtype=self.dtype, device=self.device)

    # -- loader dispatch --------------------------------------------------------------

    def get_weights(self, prefix: str):
        return self.weights_loader.get_weights(self, prefix)

    def get_weights_col_packed_qkv(self, prefix: str, num_heads: int, num_key_value_heads: int):
        return self.get_weights_col_packed(prefix, [num_heads, num_key_value_heads, num_key_value_heads])

    def get_weights_col_packed_gate_up(self, prefix: str):
        return self.get_weights_col_packed(prefix, 2)

    def get_weights_col_packed(self, prefix: str, block_sizes):
        return self.weights_loader.get_weights_col_packed(self, prefix, block_sizes)

    def get_weights_col(self, prefix: str):
        return self.weights_loader.get_weights_col(self, prefix)

    def get_multi_weights_col(self, prefixes: List[str], dim: int):
        return self.weights_loader.get_multi_weights_col(self, prefixes, dim)

    def get_weights_row(self, prefix: str):
        return self.weights_loader.get_weights_row(self, prefix)

    @contextmanager
    def use_loader(self, weights_loader: WeightsLoader):
        previous, self.weights_loader = self.weights_loader, weights_loader
        try:
            yield
        finally:
            self.weights_loader = previous

    @property
    def loader(self):
        return self.weights_loader


def _cut(source, dim: int, start: int, stop: int):
    if dim == 0:
        return source[start:stop]
    if dim == 1:
        return source[:, start:stop]
    raise NotImplementedError("only dim 0 and dim 1 can be sharded")
