"""Reading a model's weights from disk without ever widening or executing them.

Public surface as the reference's iron/lm/checkpoint.py:31-294 (``Checkpoint``, ``weights_file``,
``nest`` / ``leaves``) plus ``write_safetensors`` for toy checkpoints.  Three containers are
understood: one ``.safetensors`` file; a sharded set named by a ``.safetensors.index.json``; and a
PyTorch zip (``.pth`` / ``.bin``), whose pickle is read strictly as data.

The files are memory-mapped and a tensor costs nothing until it is asked for:

* ``Checkpoint.torch(name)`` wraps the mapped bytes in a torch tensor, bf16 staying 16-bit.  This is
  what goes to the GPU: a checkpoint streams from the page cache into HBM with no float32 copy of it
  ever existing on the host.
* ``Checkpoint.tensors[name]`` gives the host-side array of this package's convention (bf16 widened
  to bf16-valued float32), for the CPU stand-in and for tests.
"""

from __future__ import annotations

import dataclasses
import io
import json
import math
import mmap
import pickle
import struct
import zipfile
from collections import OrderedDict
from collections.abc import Iterator, Mapping
from pathlib import Path
from types import SimpleNamespace
from typing import Any

import numpy as np

from ..bf16 import bfloat16, from_bits

# safetensors dtype tag -> (element type as this package names it, numpy dtype of the stored bytes)
_SAFETENSORS_TYPES = {
    "BF16": (bfloat16, np.uint16),
    "F16": (np.float16, np.float16),
    "F32": (np.float32, np.float32),
    "I64": (np.int64, np.int64),
}
# torch storage class name -> the same pair
_TORCH_STORAGES = {
    "BFloat16Storage": _SAFETENSORS_TYPES["BF16"],
    "HalfStorage": _SAFETENSORS_TYPES["F16"],
    "FloatStorage": _SAFETENSORS_TYPES["F32"],
    "LongStorage": _SAFETENSORS_TYPES["I64"],
}
_ZIP_LOCAL_HEADER = struct.Struct("<4s5H3I2H")    # PKZIP local file header, 30 bytes


@dataclasses.dataclass(frozen=True)
class StoredTensor:
    """A tensor exactly as the file has it: a read-only view into the mapping (bf16 as uint16)."""

    view: np.ndarray
    element: Any

    @property
    def shape(self) -> tuple[int, ...]:
        return tuple(self.view.shape)

    def widened(self) -> np.ndarray:
        return from_bits(self.view) if self.element is bfloat16 else self.view


class _MappedFile:
    """One file of a checkpoint under a read-only mapping, with the tensors found in it."""

    def __init__(self, path: Path):
        self.path = path
        with open(path, "rb") as handle:
            self.mapping = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_READ)
        self.bytes = np.frombuffer(self.mapping, dtype=np.uint8)
        self.base_address = self.bytes.ctypes.data
        reader = _read_torch_zip if zipfile.is_zipfile(path) else _read_safetensors
        self.tensors: dict[str, StoredTensor] = reader(self)

    def drop_pages(self, array: np.ndarray) -> bool:
        """If ``array`` lies in this mapping, let the kernel reclaim its pages (they fault back in
        from the file if touched again).  Used after a tensor has been uploaded."""
        offset = array.ctypes.data - self.base_address
        inside = array.flags.c_contiguous and 0 <= offset < len(self.mapping)
        if inside:
            page_start = offset // mmap.PAGESIZE * mmap.PAGESIZE
            self.mapping.madvise(mmap.MADV_DONTNEED, page_start, offset + array.nbytes - page_start)
        return bool(inside)


def _read_safetensors(file: _MappedFile) -> dict[str, StoredTensor]:
    """8 bytes of little-endian header length, a JSON header, then the tensors' bytes."""
    path, total = file.path, len(file.mapping)
    if total < 8:
        raise ValueError(f"{path}: {total} bytes hold no safetensors header")
    header_bytes = struct.unpack_from("<Q", file.mapping, 0)[0]
    data_start = 8 + header_bytes
    if data_start > total:
        raise ValueError(f"{path}: a header of {header_bytes} bytes does not fit the file")
    entries = json.loads(file.mapping[8:data_start])
    entries.pop("__metadata__", None)
    found = {}
    for name, entry in entries.items():
        tag = entry.get("dtype")
        if tag not in _SAFETENSORS_TYPES:
            raise ValueError(f"{path}: {name} is {tag}")
        offsets, shape = entry.get("data_offsets"), entry.get("shape")
        if shape is None or offsets is None or len(offsets) != 2:
            raise ValueError(f"{path}: {name} has no data_offsets or shape")
        element, stored = _SAFETENSORS_TYPES[tag]
        lo, hi = data_start + offsets[0], data_start + offsets[1]
        expected = math.prod(shape) * np.dtype(stored).itemsize
        if not (data_start <= lo and hi <= total and hi - lo == expected):
            raise ValueError(f"{path}: {name} spans bytes {lo} to {hi}, not {tag} {shape} within the file")
        found[name] = StoredTensor(file.bytes[lo:hi].view(stored).reshape(shape), element)
    return found


def _read_torch_zip(file: _MappedFile) -> dict[str, StoredTensor]:
    """``torch.save``'s zip: ``<root>/data.pkl`` describes tensors as views of storages kept
    uncompressed under ``<root>/data/<key>``, so each tensor can be a view straight into the mapping."""
    archive = zipfile.ZipFile(file.path)
    members = archive.namelist()
    if not members:
        raise ValueError(f"{file.path}: an empty archive, not a checkpoint")
    root = members[0].partition("/")[0]

    def storage_bytes(key: str) -> np.ndarray:
        info = archive.getinfo(f"{root}/data/{key}")
        if info.compress_type != zipfile.ZIP_STORED:
            raise ValueError(f"{file.path}: storage {key} is compressed")
        fields = _ZIP_LOCAL_HEADER.unpack_from(file.mapping, info.header_offset)
        name_length, extra_length = fields[-2], fields[-1]
        start = info.header_offset + _ZIP_LOCAL_HEADER.size + name_length + extra_length
        return file.bytes[start : start + info.file_size]

    state = _StateDictUnpickler(io.BytesIO(archive.read(f"{root}/data.pkl")), storage_bytes).load()
    flat: dict[str, StoredTensor] = {}

    def collect(prefix: str, node) -> None:
        if isinstance(node, StoredTensor):
            flat[prefix] = node
        elif isinstance(node, dict):
            for key, child in node.items():
                collect(f"{prefix}.{key}" if prefix else str(key), child)

    collect("", state)
    return flat


class _StateDictUnpickler(pickle.Unpickler):
    """Unpickles a state dict and nothing else.

    A pickle can name any importable callable; this one resolves exactly the handful a plain state
    dict needs (an ordered dict, the tensor rebuild hook, four storage types) and refuses every other
    global before it could be called, so no code from the file or on its behalf runs.  Tensors come
    out as ``StoredTensor`` views, each checked to lie inside its storage."""

    def __init__(self, stream, storage_bytes):
        super().__init__(stream)
        self._storage_bytes = storage_bytes

    def find_class(self, module: str, name: str):
        if (module, name) == ("collections", "OrderedDict"):
            return OrderedDict
        if (module, name) == ("torch._utils", "_rebuild_tensor_v2"):
            return self._tensor_view
        if module == "torch" and name in _TORCH_STORAGES:
            return _TORCH_STORAGES[name]
        raise pickle.UnpicklingError(f"a checkpoint may not load {module}.{name}")

    def persistent_load(self, pid):
        """torch pickles a storage as the persistent id ``("storage", type, key, location, numel)``."""
        well_formed = (isinstance(pid, tuple) and len(pid) == 5 and pid[0] == "storage"
                       and any(pid[1] is pair for pair in _TORCH_STORAGES.values())
                       and isinstance(pid[2], str) and isinstance(pid[4], int))
        if not well_formed:
            raise pickle.UnpicklingError(f"a checkpoint's storage id is {pid!r}")
        (element, stored), key, count = pid[1], pid[2], pid[4]
        raw = self._storage_bytes(key)
        wanted = count * np.dtype(stored).itemsize
        if count < 0 or wanted > raw.size:
            raise pickle.UnpicklingError(f"storage {key} holds {raw.size} bytes, not {count} {np.dtype(stored)}")
        return StoredTensor(raw[:wanted].view(stored), element)

    @staticmethod
    def _tensor_view(storage, offset, size, stride, *_ignored):
        """Stand-in for ``torch._utils._rebuild_tensor_v2``: a strided read-only window of a storage."""
        numbers = (offset, *size, *stride) if isinstance(size, tuple) and isinstance(stride, tuple) else (None,)
        if not (isinstance(storage, StoredTensor) and len(size) == len(stride)
                and all(isinstance(n, int) and n >= 0 for n in numbers)):
            raise pickle.UnpicklingError("a checkpoint's tensor is not one")
        elements = storage.view
        if math.prod(size):
            furthest = offset + sum((extent - 1) * step for extent, step in zip(size, stride))
            if furthest >= elements.size:
                raise pickle.UnpicklingError(f"a tensor reaches element {furthest} of a {elements.size}-element storage")
        byte_strides = tuple(step * elements.itemsize for step in stride)
        window = np.lib.stride_tricks.as_strided(elements[offset:], shape=size, strides=byte_strides, writeable=False)
        return StoredTensor(window, storage.element)


def weights_file(directory) -> Path:
    """Which file of a checkpoint directory to open: the shard index when there is one, else the
    single ``model.safetensors``."""
    folder = Path(directory)
    index = folder / "model.safetensors.index.json"
    return index if index.exists() else folder / "model.safetensors"


class _HostView(Mapping):
    """``name -> host array`` over stored tensors, widening on access only."""

    def __init__(self, stored: dict[str, StoredTensor]):
        self._stored = stored

    def __getitem__(self, name: str) -> np.ndarray:
        return self._stored[name].widened()

    def __iter__(self) -> Iterator[str]:
        return iter(self._stored)

    def __len__(self) -> int:
        return len(self._stored)


class Checkpoint:
    """Every tensor of a checkpoint under one roof, whichever container holds it.  Pass a
    ``.safetensors`` file, a PyTorch zip, or a shard index (``*.safetensors.index.json``): the
    shards the index names must sit beside it and hold exactly the tensors it assigns to them."""

    def __init__(self, path):
        self.path = Path(path)
        assignment = None          # tensor name -> shard file name, for a sharded checkpoint
        files = [self.path]
        if self.path.suffix == ".json":
            assignment = json.loads(self.path.read_text())["weight_map"]
            shard_names = sorted(set(assignment.values()))
            outside = [n for n in shard_names if Path(n).name != n]
            if outside:
                raise ValueError(f"{self.path}: {outside[0]} is not a file beside the index")
            files = [self.path.with_name(n) for n in shard_names]
        self._files = [_MappedFile(f) for f in files]
        self._stored: dict[str, StoredTensor] = {}
        for file in self._files:
            if assignment is not None:
                promised = {name for name, shard in assignment.items() if shard == file.path.name}
                present = set(file.tensors)
                if promised != present:
                    raise ValueError(f"{file.path}: holds {sorted(present - promised)} the index does not name "
                                     f"and lacks {sorted(promised - present)}")
            self._stored.update(file.tensors)
        self.tensors: Mapping[str, np.ndarray] = _HostView(self._stored)

    def shapes(self) -> dict[str, tuple[tuple[int, ...], Any]]:
        """``name -> (shape, element type)`` without touching any tensor's bytes."""
        return {name: (t.shape, t.element) for name, t in self._stored.items()}

    def torch(self, name: str):
        """The stored bytes as a torch tensor (zero-copy when contiguous; bf16 stays bf16)."""
        import warnings

        import torch

        stored = self._stored[name]
        array = stored.view if stored.view.flags.c_contiguous else np.ascontiguousarray(stored.view)
        with warnings.catch_warnings():
            # torch warns that the array is not writable; nothing downstream writes through it
            warnings.simplefilter("ignore", UserWarning)
            tensor = torch.from_numpy(array)
        return tensor.view(torch.bfloat16) if stored.element is bfloat16 else tensor

    def state_dict(self, *, as_torch: bool = False) -> dict[str, Any]:
        """All tensors by name, as ``torch()`` gives them or as host arrays."""
        pick = self.torch if as_torch else self.tensors.__getitem__
        return {name: pick(name) for name in self._stored}

    def release(self, array: np.ndarray) -> None:
        """Give back the resident pages behind ``array`` if it views one of this checkpoint's files."""
        any(file.drop_pages(array) for file in self._files)

    def tree(self) -> SimpleNamespace:
        """The host arrays arranged by dotted name (``model.layers.3.x`` -> ``tree.model.layers[3].x``)."""
        return nest({name: self.tensors[name] for name in self._stored}, file=self.path)


# ---- dotted names <-> nested objects


def leaves(tree, prefix: str = "") -> Iterator[tuple[str, Any]]:
    """Walk a tree built by ``nest`` back into ``(dotted name, value)`` pairs."""
    if isinstance(tree, list):
        children = [(str(i), child) for i, child in enumerate(tree)]
    elif isinstance(tree, SimpleNamespace):
        children = list(vars(tree).items())
    else:
        yield prefix.rstrip("."), tree
        return
    for key, child in children:
        yield from leaves(child, f"{prefix}{key}.")


def nest(named: Mapping[str, Any], path: str = "", file: str | Path = "the checkpoint"):
    """Turn ``{"a.b.0.w": v, ...}`` into attribute access; components that are all numbers become a
    list (holes, i.e. modules without tensors of their own, come out as empty modules)."""
    root: dict = {}
    for dotted, value in named.items():
        cursor = root
        parts = dotted.split(".")
        for part in parts[:-1]:
            cursor = cursor.setdefault(part, {})
        cursor[parts[-1]] = value
    return _build(root, path, file)


def _build(node, path: str, file):
    if not isinstance(node, dict):
        return node
    children = {key: _build(child, f"{path}{key}.", file) for key, child in node.items()}
    if children and all(key.isdigit() for key in children):
        highest = max(int(key) for key in children)
        # Holes are modules without weights (an activation between two layers): a few at most.  An
        # index far beyond what is present is a damaged or foreign file, not a list to pad out.
        if highest + 1 > 2 * len(children) + 8:
            raise ValueError(f"{file}: {path}{highest} is past its {len(children)} layers")
        built = _ModuleList(children.get(str(i), _build({}, f"{path}{i}.", file)) for i in range(highest + 1))
    else:
        built = _Module(**children)
    built._path, built._file = path, file
    return built


class _Module(SimpleNamespace):
    """Attribute access over a module's children; a missing one says where it was looked for."""

    __slots__ = ("_path", "_file")

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        have = ", ".join(vars(self)) or "nothing"
        raise AttributeError(f"{self._path}{name} is not in {self._file} (it has {have})")


class _ModuleList(list):
    """Index access over numbered modules; an index past the end says so with the full path."""

    __slots__ = ("_path", "_file")

    def __getitem__(self, index):
        if isinstance(index, int) and not -len(self) <= index < len(self):
            raise IndexError(f"{self._path}{index} is not in {self._file} (it has {len(self)})")
        return super().__getitem__(index)


def write_safetensors(path, tensors: Mapping[str, np.ndarray], dtypes: Mapping[str, str] | None = None) -> Path:
    """Save host arrays as one ``.safetensors`` file.  A float32 array whose values are all
    bf16-representable is stored as ``BF16`` (2 bytes an element) unless ``dtypes[name]`` says
    otherwise; float16 and int64 keep their type."""
    from ..bf16 import is_bf16_valued, to_bits

    chosen = dict(dtypes or {})
    directory, payload, cursor = {}, [], 0
    for name, value in tensors.items():
        array = np.asarray(value)
        tag = chosen.get(name)
        if tag is None:
            if array.dtype == np.float16:
                tag = "F16"
            elif array.dtype == np.int64:
                tag = "I64"
            else:
                tag = "BF16" if is_bf16_valued(array) else "F32"
        if tag == "BF16":
            data = to_bits(array).tobytes()
        else:
            data = np.ascontiguousarray(array, dtype=_SAFETENSORS_TYPES[tag][1]).tobytes()
        directory[name] = {"dtype": tag, "shape": list(array.shape), "data_offsets": [cursor, cursor + len(data)]}
        payload.append(data)
        cursor += len(data)
    header = json.dumps(directory).encode()
    header += b" " * (-len(header) % 8)        # keep the tensor data 8-byte aligned
    target = Path(path)
    with open(target, "wb") as out:
        out.write(struct.pack("<Q", len(header)))
        out.write(header)
        out.writelines(payload)
    return target
