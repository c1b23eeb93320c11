"""Reading and writing safetensors files: an 8-byte little-endian header length, a
JSON header {name: {dtype, shape, data_offsets}}, then the tensors' bytes.  The
reference loads every *.safetensors file of a folder into one map by name
(src/models/turbo_generic.rs:2039-2053); so does `open_folder` here, but lazily:
a tensor's bytes are only touched (through a memory map) when it is asked for.
"""
import json
import mmap
import os
import struct
import warnings

import torch

DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
          "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
          "BOOL": torch.bool}
NAMES = {v: k for k, v in DTYPES.items()}


class WeightFileError(ValueError):
    pass


class StoredTensor:
    """A tensor inside a file: name, dtype, shape, and a way to read it."""

    def __init__(self, file, name, dtype, shape, begin, end):
        self.file, self.name, self.dtype, self.shape, self.begin, self.end = file, name, dtype, tuple(shape), begin, end

    def read(self):
        """The tensor as a CPU tensor that views the file's memory map (do not write to it)."""
        count = 1
        for s in self.shape:
            count *= s
        if count == 0:
            return torch.empty(self.shape, dtype=self.dtype)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the map is read-only; it is only copied from
            flat = torch.frombuffer(self.file.map, dtype=self.dtype, count=count, offset=self.file.data_start + self.begin)
        return flat.reshape(self.shape)


class SafetensorsFile:
    def __init__(self, path):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise WeightFileError("Cannot read %s: %s" % (path, e))
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise WeightFileError("%s: too short to be a safetensors file" % path)
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise WeightFileError("%s: header length %d exceeds the file" % (path, n))
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except ValueError as e:
            raise WeightFileError("%s: invalid header: %s" % (path, e))
        self.data_start = 8 + n
        self.map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.tensors = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            if info["dtype"] not in DTYPES:
                raise WeightFileError("%s: tensor %s has unsupported dtype %s" % (path, name, info["dtype"]))
            begin, end = info["data_offsets"]
            if not (0 <= begin <= end <= size - self.data_start):
                raise WeightFileError("%s: tensor %s lies outside the file" % (path, name))
            self.tensors[name] = StoredTensor(self, name, DTYPES[info["dtype"]], info["shape"], begin, end)


def open_folder(model_dir):
    """name -> StoredTensor over every *.safetensors file of the folder."""
    try:
        files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    except OSError as e:
        raise WeightFileError("Cannot read model dir: %s" % e)
    if not files:
        raise WeightFileError("No .safetensors files found in %s" % model_dir)
    tensors = {}
    for f in files:
        tensors.update(SafetensorsFile(os.path.join(model_dir, f)).tensors)
    return tensors


def write_file(path, tensors, metadata=None):
    """Write name -> CPU tensor as one safetensors file; `tensors` may be an iterable of
    (name, tensor) made on the fly, each tensor is written and dropped in turn."""
    items = []
    offset = 0
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    tmp = path + ".data%d" % os.getpid()
    with open(tmp, "wb") as data:
        for name, t in (tensors.items() if isinstance(tensors, dict) else tensors):
            t = t.detach().cpu().contiguous()
            raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
            header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
            data.write(raw)
            offset += len(raw)
            items.append(name)
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as out, open(tmp, "rb") as data:
        out.write(struct.pack("<Q", len(blob)))
        out.write(blob)
        while True:
            chunk = data.read(1 << 24)
            if not chunk:
                break
            out.write(chunk)
    os.remove(tmp)
    return items
