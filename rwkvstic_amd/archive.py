"""Reading the tensors of a TorchScript archive without running anything stored in it.

The reference exports its quantised model with ``torch.jit.save`` (reference
src/rwkvstic/agnostic/backends/opt.py:112-117) and loads it back with ``torch.jit.load`` (opt.py:89-92), which
compiles and later runs the code kept in the archive.  The tensors themselves sit in the archive as plain data:

* ``<name>/data.pkl`` - a pickle of the module object: every scripted object is a class named
  ``__torch__....`` created with an empty argument tuple and filled from a dict of its attributes (sub-modules are
  attributes too; the entries of a ``ModuleList`` are called "0", "1", ...); every tensor is a call of
  ``torch._utils._rebuild_tensor_v2`` on a storage that is named by a persistent id
  ``("storage", <storage type>, <key>, <device>, <numel>)``;
* ``<name>/data/<key>`` - the raw bytes of that storage (little endian).

``read_archive_tensors`` unpickles ``data.pkl`` with an unpickler that resolves only those names - scripted classes
become inert attribute holders, nothing else is importable - and returns the flat ``{attribute path: tensor}`` dict
that ``HipRWKV.from_quantized`` takes: for an export of the reference's FASTQUANT model that is the attribute tree of
``myRWKV`` (opt.py:31-48: ``emptyState``, ``emb.w``, ``ln_in/ln_out.{weight,bias}``, ``head.weights.0.*``,
``blocks.i.*`` with block.py:13-47 and matmul.py:12,67-68 below it).

No export of the reference itself exists to test against (it cannot be run here), so agreement with a real
``.rwkv`` file is untested; the reader is tested on archives that carry that attribute tree as plain tensor
attributes of scripted modules, which is how the reference's modules hold them.
"""
from __future__ import annotations

import collections
import pickle
import zipfile
from typing import Dict

import torch

_STORAGE_DTYPES = {
    "DoubleStorage": torch.float64, "FloatStorage": torch.float32, "HalfStorage": torch.float16,
    "BFloat16Storage": torch.bfloat16, "LongStorage": torch.int64, "IntStorage": torch.int32,
    "ShortStorage": torch.int16, "CharStorage": torch.int8, "ByteStorage": torch.uint8, "BoolStorage": torch.bool,
}


class _StorageType:
    def __init__(self, dtype: torch.dtype):
        self.dtype = dtype


class ScriptObject:
    """Inert stand-in for an object of a scripted class: holds the attribute dict, has no behaviour."""

    qualified_name = ""

    def __setstate__(self, state):
        if isinstance(state, dict):
            self.__dict__.update(state)
        else:                                   # a class with its own __getstate__: kept, not interpreted
            self.__dict__["__state__"] = state


def _rebuild_tensor(storage, offset, size, stride, requires_grad=False, hooks=None, metadata=None):
    size, stride = tuple(int(s) for s in size), tuple(int(s) for s in stride)
    need = int(offset) + 1 + sum((n - 1) * s for n, s in zip(size, stride)) if all(n > 0 for n in size) else 0
    if any(s < 0 for s in stride) or int(offset) < 0 or need > storage.numel():
        raise pickle.UnpicklingError("tensor view outside its storage")
    return torch.as_strided(storage, size, stride, int(offset))


def _passthrough(x):
    return x


class _Unpickler(pickle.Unpickler):
    def __init__(self, file, zf: zipfile.ZipFile, root: str):
        super().__init__(file)
        self.zf, self.root = zf, root
        self.storages: Dict[str, torch.Tensor] = {}
        self.classes: Dict[str, type] = {}

    def find_class(self, module: str, name: str):
        if module == "__torch__" or module.startswith("__torch__."):
            q = f"{module}.{name}"
            if q not in self.classes:
                self.classes[q] = type(name, (ScriptObject,), {"qualified_name": q})
            return self.classes[q]
        if module == "torch._utils" and name in ("_rebuild_tensor_v2", "_rebuild_tensor"):
            return _rebuild_tensor
        if module == "torch" and name in _STORAGE_DTYPES:
            return _StorageType(_STORAGE_DTYPES[name])
        if module == "torch" and name == "device":
            return str                              # torch.device("cuda:0") -> its name, nothing is moved here
        if module == "collections" and name == "OrderedDict":
            return collections.OrderedDict
        if module == "torch.jit._pickle" and (name.startswith("build_") or name == "restore_type_tag"):
            return (lambda x, *_: x) if name == "restore_type_tag" else _passthrough
        raise pickle.UnpicklingError(f"archive refers to {module}.{name}: not something a tensor archive needs")

    def persistent_load(self, pid):
        if not (isinstance(pid, tuple) and len(pid) >= 5 and pid[0] == "storage" and isinstance(pid[1], _StorageType)):
            raise pickle.UnpicklingError(f"unknown persistent id {pid!r}")
        dtype, key, numel = pid[1].dtype, str(pid[2]), int(pid[4])
        if key not in self.storages:
            raw = bytearray(self.zf.read(f"{self.root}/data/{key}"))
            item = torch.empty((), dtype=dtype).element_size()
            if len(raw) < numel * item:
                raise pickle.UnpicklingError(f"storage {key}: {len(raw)} bytes for {numel} elements of {dtype}")
            self.storages[key] = (torch.frombuffer(raw, dtype=dtype, count=numel) if numel
                                  else torch.empty(0, dtype=dtype))
        return self.storages[key]


def read_archive_object(path: str):
    """The unpickled module object of a ``torch.jit.save`` archive as a tree of :class:`ScriptObject`."""
    with zipfile.ZipFile(path) as zf:
        roots = [n[: -len("/data.pkl")] for n in zf.namelist() if n.endswith("/data.pkl") and n.count("/") == 1]
        if len(roots) != 1:
            raise ValueError(f"{path}: not a torch.jit archive (found {len(roots)} data.pkl records)")
        with zf.open(roots[0] + "/data.pkl") as f:
            return _Unpickler(f, zf, roots[0]).load()


def read_archive_tensors(path: str) -> Dict[str, torch.Tensor]:
    """``{dotted attribute path: CPU tensor}`` of every tensor reachable through module attributes (lists and dicts of
    tensors are indexed by position / key).  Nothing of the archive's code is compiled or run."""
    out: Dict[str, torch.Tensor] = {}
    seen = set()

    def walk(prefix: str, obj) -> None:
        if isinstance(obj, torch.Tensor):
            out[prefix] = obj
        elif isinstance(obj, ScriptObject):
            if id(obj) in seen:
                return
            seen.add(id(obj))
            for k, v in obj.__dict__.items():
                walk(f"{prefix}.{k}" if prefix else str(k), v)
        elif isinstance(obj, (list, tuple)):
            for i, v in enumerate(obj):
                walk(f"{prefix}.{i}" if prefix else str(i), v)
        elif isinstance(obj, dict):
            for k, v in obj.items():
                walk(f"{prefix}.{k}" if prefix else str(k), v)

    walk("", read_archive_object(path))
    return out
