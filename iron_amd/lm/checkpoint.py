"""A model's weights read from its checkpoint: ``Checkpoint(path).tensors``, by their own names.

A ``.safetensors`` file, a sharded checkpoint given by its ``.safetensors.index.json``, or a
PyTorch checkpoint (a ``.pth`` / ``.bin`` zip, read as data through a whitelisting unpickler that
runs no code of the file's) -- iron/lm/checkpoint.py:31-294.  Files are memory-mapped; a tensor
is materialised when it is asked for:

* ``tensors[name]``: a host array in this package's convention -- bf16 as a bf16-valued float32
  array (``iron_amd.bf16``), f16/f32/i64 as numpy's own;
* ``torch(name)``: a torch tensor over the mapped bytes (bf16 stays 2 bytes), what
  ``load_state_dict`` takes as it is, so a 1B checkpoint is never widened on the host.
"""

from __future__ import annotations

import io
import json
import math
import mmap
import pickle
import struct
import zipfile
from collections import OrderedDict
from collections.abc import Callable, Iterator, Mapping
from pathlib import Path
from types import SimpleNamespace
from typing import Any

import numpy as np

from ..bf16 import bfloat16, from_bits


class _Raw:
    """A tensor as the file holds it: a read-only numpy view, bf16 as its uint16 storage."""

    __slots__ = ("bits", "dtype")

    def __init__(self, bits: np.ndarray, dtype):
        self.bits, self.dtype = bits, dtype

    @property
    def shape(self) -> tuple[int, ...]:
        return tuple(self.bits.shape)

    def host(self) -> np.ndarray:
        return from_bits(self.bits) if self.dtype is bfloat16 else self.bits


class _Shard:
    """One ``.safetensors`` file or one PyTorch zip, mapped; ``raw`` are lazy views of it."""

    # name in the file's header -> (element type, numpy type of the mapped bytes)
    DTYPES = {"BF16": (bfloat16, np.uint16), "F16": (np.float16, np.float16), "F32": (np.float32, np.float32),
              "I64": (np.int64, np.int64)}

    def __init__(self, path: Path):
        self.path = path
        with open(path, "rb") as f:
            self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)  # keeps its own reference to the file
        data = np.frombuffer(self._map, dtype=np.uint8)
        self._address = data.ctypes.data
        if zipfile.is_zipfile(path):
            self.raw = self._torch(data)
            return
        if len(self._map) < 8:
            raise ValueError(f"{path}: {len(self._map)} bytes hold no safetensors header")
        (length,) = struct.unpack("<Q", self._map[:8])
        if 8 + length > len(self._map):
            raise ValueError(f"{path}: a header of {length} bytes does not fit the file")
        header = json.loads(self._map[8 : 8 + length])
        header.pop("__metadata__", None)
        self.raw: dict[str, _Raw] = {}
        for name, t in header.items():
            if t.get("dtype") not in self.DTYPES:
                raise ValueError(f"{path}: {name} is {t.get('dtype')}")
            if len(t.get("data_offsets", ())) != 2 or "shape" not in t:
                raise ValueError(f"{path}: {name} has no data_offsets or shape")
            begin, end = (8 + length + o for o in t["data_offsets"])
            element, stored = self.DTYPES[t["dtype"]]
            if (end - begin != np.dtype(stored).itemsize * math.prod(t["shape"]) or begin < 8 + length
                    or end > data.size):
                raise ValueError(f"{path}: {name} spans bytes {begin} to {end}, not {t['dtype']} {t['shape']} "
                                 "within the file")
            self.raw[name] = _Raw(data[begin:end].view(stored).reshape(t["shape"]), element)

    def _torch(self, data: np.ndarray) -> dict[str, _Raw]:
        """A PyTorch checkpoint's tensors, each a view of its storage's bytes (stored uncompressed)."""
        archive = zipfile.ZipFile(self.path)
        if not archive.namelist():
            raise ValueError(f"{self.path}: an empty archive, not a checkpoint")
        root = archive.namelist()[0].split("/")[0]

        def storage(key: str) -> np.ndarray:
            info = archive.getinfo(f"{root}/data/{key}")
            if info.compress_type != zipfile.ZIP_STORED:
                raise ValueError(f"{self.path}: storage {key} is compressed")
            # A ZIP local file header is 30 bytes with its name's and extra field's lengths at 26.
            header, lengths = info.header_offset + 30, info.header_offset + 26
            begin = header + sum(struct.unpack("<HH", self._map[lengths:header]))
            return data[begin : begin + info.file_size]

        state = _TorchUnpickler(io.BytesIO(archive.read(f"{root}/data.pkl")), storage).load()
        tensors, pending = {}, [("", state)]
        while pending:
            path, node = pending.pop()
            if isinstance(node, _Raw):
                tensors[path] = node
            elif isinstance(node, dict):
                pending += [(f"{path}.{k}" if path else k, v) for k, v in node.items()]
        return tensors

    def release(self, array: np.ndarray) -> bool:
        """Drop the process's pages of ``array`` if it views this file (it stays readable)."""
        begin = array.ctypes.data - self._address
        if not (array.flags.c_contiguous and 0 <= begin < len(self._map)):
            return False
        start = begin - begin % mmap.PAGESIZE
        self._map.madvise(mmap.MADV_DONTNEED, start, begin + array.nbytes - start)
        return True


class _TorchUnpickler(pickle.Unpickler):
    """A state dict's pickle read as data: ``GLOBALS`` names every global it may use, so loading one
    runs no code of the file's; each tensor becomes a view of its storage, checked to lie inside it."""

    GLOBALS = {
        ("collections", "OrderedDict"): OrderedDict,
        ("torch._utils", "_rebuild_tensor_v2"): None,
        ("torch", "BFloat16Storage"): (bfloat16, np.uint16),
        ("torch", "HalfStorage"): (np.float16, np.float16),
        ("torch", "FloatStorage"): (np.float32, np.float32),
        ("torch", "LongStorage"): (np.int64, np.int64),
    }

    def __init__(self, file, storage: Callable[[str], np.ndarray]):
        super().__init__(file)
        self.storage = storage

    def find_class(self, module: str, name: str):
        if (module, name) not in self.GLOBALS:
            raise pickle.UnpicklingError(f"a checkpoint may not load {module}.{name}")
        if (module, name) == ("torch._utils", "_rebuild_tensor_v2"):
            return self.rebuild
        return self.GLOBALS[module, name]

    def persistent_load(self, pid):
        """A storage by its key: ``("storage", dtype, key, location, numel)``."""
        kinds = [d for (_, name), d in self.GLOBALS.items() if name.endswith("Storage")]
        if not (isinstance(pid, tuple) and len(pid) == 5 and pid[0] == "storage" and any(pid[1] is d for d in kinds)
                and isinstance(pid[2], str) and isinstance(pid[4], int)):
            raise pickle.UnpicklingError(f"a checkpoint's storage id is {pid!r}")
        _, (element, stored), key, _, numel = pid
        data, size = self.storage(key), np.dtype(stored).itemsize
        if not 0 <= numel * size <= data.size:
            raise pickle.UnpicklingError(f"storage {key} holds {data.size} bytes, not {numel} {np.dtype(stored)}")
        return _Raw(data[: numel * size].view(stored), element)

    @staticmethod
    def rebuild(storage, offset, size, stride, *_):
        """``torch._utils._rebuild_tensor_v2``'s tensor as a read-only view of ``storage``."""
        if not (isinstance(storage, _Raw) and isinstance(size, tuple) and isinstance(stride, tuple)
                and len(size) == len(stride)
                and all(isinstance(n, int) and n >= 0 for n in (offset, *size, *stride))):
            raise pickle.UnpicklingError("a checkpoint's tensor is not one")
        bits = storage.bits
        last = offset + sum((n - 1) * s for n, s in zip(size, stride) if n)
        if math.prod(size) and last >= bits.size:
            raise pickle.UnpicklingError(f"a tensor reaches element {last} of a {bits.size}-element storage")
        view = np.lib.stride_tricks.as_strided(bits[offset:], size, tuple(s * bits.itemsize for s in stride),
                                               writeable=False)
        return _Raw(view, storage.dtype)


def weights_file(directory) -> Path:
    """A checkpoint directory's weights file: the sharded index if there is one, else ``model.safetensors``."""
    index = Path(directory) / "model.safetensors.index.json"
    return index if index.exists() else index.with_name("model.safetensors")


class _Tensors(Mapping):
    """``name -> host array``, converted when asked for (a bf16 tensor widens to float32 then)."""

    def __init__(self, raw: dict[str, _Raw]):
        self._raw = raw

    def __getitem__(self, name: str) -> np.ndarray:
        return self._raw[name].host()

    def __iter__(self) -> Iterator[str]:
        return iter(self._raw)

    def __len__(self) -> int:
        return len(self._raw)


class Checkpoint:
    """A ``.safetensors`` file or a PyTorch checkpoint -- or, given its ``.safetensors.index.json``,
    every shard a sharded checkpoint splits across, merged into one mapping."""

    def __init__(self, path):
        self.path = Path(path)
        weight_map = None
        paths = [self.path]
        if self.path.suffix == ".json":
            weight_map = json.loads(self.path.read_text())["weight_map"]
            names = sorted(set(weight_map.values()))
            for n in names:
                if Path(n).name != n:
                    raise ValueError(f"{self.path}: {n} is not a file beside the index")
            paths = [self.path.parent / n for n in names]
        self._shards = [_Shard(p) for p in paths]
        self._raw: dict[str, _Raw] = {}
        for shard in self._shards:
            if weight_map is not None:
                named = {n for n, s in weight_map.items() if s == shard.path.name}
                if named != shard.raw.keys():
                    raise ValueError(f"{shard.path}: holds {sorted(shard.raw.keys() - named)} the index does not "
                                     f"name and lacks {sorted(named - shard.raw.keys())}")
            self._raw.update(shard.raw)
        self.tensors: Mapping[str, np.ndarray] = _Tensors(self._raw)

    def shapes(self) -> dict[str, tuple[tuple[int, ...], Any]]:
        """Each tensor's ``(shape, element type)`` by name, from the headers alone."""
        return {n: (r.shape, r.dtype) for n, r in self._raw.items()}

    def torch(self, name: str):
        """``name`` as a torch tensor over the mapped bytes: bf16 stays bf16 (2 bytes an element)."""
        import warnings

        import torch

        raw = self._raw[name]
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)  # the mapping is read-only; nothing here writes it
            t = torch.from_numpy(np.ascontiguousarray(raw.bits) if not raw.bits.flags.c_contiguous else raw.bits)
        return t.view(torch.bfloat16) if raw.dtype is bfloat16 else t

    def state_dict(self, *, as_torch: bool = False) -> dict[str, Any]:
        """Every tensor by name: torch tensors over the file (``as_torch``) or host arrays."""
        return {n: (self.torch(n) if as_torch else self.tensors[n]) for n in self._raw}

    def release(self, array: np.ndarray) -> None:
        """Drop the process's pages of ``array`` if it views one of the files."""
        for shard in self._shards:
            if shard.release(array):
                return

    def tree(self) -> SimpleNamespace:
        """The tensors nested by their dotted names: ``model.layers.3.x`` is ``tree.model.layers[3].x``."""
        return nest(dict(self.tensors.items()), file=self.path)


def leaves(tree, prefix: str = "") -> Iterator[tuple[str, Any]]:
    """Each leaf of a nested tree by its dotted name: ``nest``'s inverse."""
    if isinstance(tree, (list, SimpleNamespace)):
        items = enumerate(tree) if isinstance(tree, list) else vars(tree).items()
        for name, value in items:
            yield from leaves(value, f"{prefix}{name}.")
    else:
        yield prefix[:-1], tree


def nest(named: Mapping[str, Any], path: str = "", file: str | Path = "the checkpoint"):
    """Nest values by dotted name; a run of modules keyed by indices becomes a list."""
    nested: dict = {}
    for name, value in named.items():
        *parents, leaf = name.split(".")
        node = nested
        for key in parents:
            node = node.setdefault(key, {})
        node[leaf] = value
    return _tree(nested, path, file)


def _tree(node, path: str, file):
    if not isinstance(node, dict):
        return node
    items = {key: _tree(child, f"{path}{key}.", file) for key, child in node.items()}
    if items and all(key.isdigit() for key in items):
        top = max(map(int, items))
        # A skipped index is a module without weights, never most of them.
        if top >= 4 * len(items) + 4:
            raise ValueError(f"{file}: {path}{top} is past its {len(items)} layers")
        tree = _Layers(items[str(i)] if str(i) in items else _tree({}, f"{path}{i}.", file) for i in range(top + 1))
    else:
        tree = _Module(**items)
    tree._path, tree._file = path, file
    return tree


class _Module(SimpleNamespace):
    """A module of a tree; a name it lacks raises naming its dotted path, the file and what it has."""

    __slots__ = ("_path", "_file")

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        raise AttributeError(f"{self._path}{name} is not in {self._file} (it has {', '.join(vars(self)) or 'nothing'})")


class _Layers(list):
    """A run of modules by index; an index past the end raises naming its path and how many there are."""

    __slots__ = ("_path", "_file")

    def __getitem__(self, index):
        try:
            return super().__getitem__(index)
        except IndexError:
            raise IndexError(f"{self._path}{index} is not in {self._file} (it has {len(self)})") from None


def write_safetensors(path, tensors: Mapping[str, np.ndarray], dtypes: Mapping[str, str] | None = None) -> Path:
    """Write host arrays as one ``.safetensors`` file (a float32 array of a bf16 tensor goes out as
    ``BF16`` unless ``dtypes`` says ``F32``): what a toy checkpoint or an exported model needs."""
    from ..bf16 import is_bf16_valued, to_bits

    header, blobs, end = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a)
        kind = (dtypes or {}).get(name)
        if kind is None:
            kind = {"float16": "F16", "int64": "I64"}.get(a.dtype.name, "BF16" if is_bf16_valued(a) else "F32")
        if kind == "BF16":
            blob = to_bits(a).tobytes()
        else:
            blob = np.ascontiguousarray(a, dtype=_Shard.DTYPES[kind][1]).tobytes()
        header[name] = {"dtype": kind, "shape": list(a.shape), "data_offsets": [end, end + len(blob)]}
        blobs.append(blob)
        end += len(blob)
    text = json.dumps(header).encode()
    text += b" " * (-len(text) % 8)
    path = Path(path)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text)
        for blob in blobs:
            f.write(blob)
    return path
