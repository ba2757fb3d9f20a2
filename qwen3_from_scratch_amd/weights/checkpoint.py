"""Weights from safetensors, by tensor name.

The reference loads every tensor of every shard into host memory and looks
names up in a dict; a missing name is a bare KeyError and unused names are never
reported (src/qwen3_from_scratch/models/parameter_loader.py:8-48). Here tensors
are read one at a time, straight to the device, and the whole set of names and
shapes is checked before the first byte is read.
"""

import glob
import json
import os

import torch


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs. One message lists
    every missing tensor, every unexpected tensor and every wrong shape."""

    def __init__(self, missing, unexpected, wrong_shape, where=""):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        lines = ["checkpoint %s does not match the model:" % where]
        if self.missing:
            lines.append("  missing tensors (%d):" % len(self.missing))
            lines += ["    " + n for n in self.missing]
        if self.unexpected:
            lines.append("  unexpected tensors (%d):" % len(self.unexpected))
            lines += ["    " + n for n in self.unexpected]
        if self.wrong_shape:
            lines.append("  wrong shapes (%d):" % len(self.wrong_shape))
            lines += [
                "    %s: expected %s, found %s" % (n, list(e), list(f))
                for n, e, f in self.wrong_shape
            ]
        super().__init__("\n".join(lines))


_KEPT = {
    torch.bfloat16: torch.bfloat16,
    torch.float32: torch.float32,
    torch.float16: torch.float32,      # every float16 number is a float32 number: nothing is rounded here
    torch.float64: torch.float32,
    torch.int32: torch.int32,
    torch.int64: torch.int32,
    torch.int16: torch.int32,
    torch.int8: torch.int32,
    torch.uint8: torch.int32,
}


def stored_to_kept(tensor, name="tensor"):
    """bfloat16 stays bfloat16, a 32-bit float tensor stays so, float16 and
    float64 tensors become float32 (the reference keeps whatever the file holds,
    src/qwen3_from_scratch/models/parameter_loader.py:35-41; the parts then bring
    matrices to the engine's compute dtype, which is bfloat16 or float32), integer
    tables become int32; anything else (8-bit floats, complex, bool) is refused."""
    if tensor.dtype not in _KEPT:
        raise ValueError(
            "%s is stored as %s; only bfloat16, float16, float32, float64 and integer tensors are loaded"
            % (name, tensor.dtype)
        )
    return tensor.to(_KEPT[tensor.dtype])


class TensorSource:
    """What a model is loaded from: names, shapes, and tensors on request."""

    where = "<source>"

    def names(self):
        raise NotImplementedError

    def shape(self, name):
        raise NotImplementedError

    def get(self, name, device):
        """The tensor in its kept dtype on `device`."""
        raise NotImplementedError


class Checkpoint(TensorSource):
    """A model folder's safetensors: `model.safetensors`, or shards listed by
    `model.safetensors.index.json`, or `model*.safetensors` shards."""

    def __init__(self, model_dir):
        from safetensors import safe_open

        self.where = model_dir
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        if os.path.isfile(index):
            with open(index) as fh:
                files = sorted(set(json.load(fh)["weight_map"].values()))
            files = [os.path.join(model_dir, f) for f in files]
        elif os.path.isfile(single):
            files = [single]
        else:
            files = sorted(glob.glob(os.path.join(model_dir, "model*.safetensors")))
        if not files:
            raise FileNotFoundError("no model.safetensors (or shards) in %s" % model_dir)
        self._handles = []
        self._file_of = {}
        for path in files:
            handle = safe_open(path, framework="pt", device="cpu")
            self._handles.append(handle)
            for name in handle.keys():
                self._file_of[name] = handle

    def names(self):
        return list(self._file_of)

    def shape(self, name):
        return tuple(self._file_of[name].get_slice(name).get_shape())

    def get(self, name, device):
        tensor = stored_to_kept(self._file_of[name].get_tensor(name), name)
        return tensor.to(device)


def check_tensors(source, expected, ignorable=()):
    """Compare the names and shapes `source` holds with `expected`
    ({name: shape}); raise one WeightError that lists every difference.
    Names in `ignorable` may be present without being expected."""
    have = set(source.names())
    want = set(expected)
    missing = want - have
    unexpected = have - want - set(ignorable)
    wrong = []
    for name in want & have:
        found = tuple(source.shape(name))
        if found != tuple(expected[name]):
            wrong.append((name, tuple(expected[name]), found))
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, source.where)
