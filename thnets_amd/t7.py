"""Torch7 binary serialisation: a writer (and a small reader) in pure Python.

The reference loads Torch7 model directories (``model.net`` + ``stat.t7``,
thapi.c:244-333, thload.c) but ships no model file, and no Lua runs here, so this
module writes such files from numpy weights: model fixtures for the tests of
``THLoadNetwork`` and a way to hand a network built in Python to the C command
line tool.  The layout is Torch7's ``torch.save(path, obj)`` in binary mode:

    object := int32 tag
      0 nil | 1 number (float64) | 2 string (int32 n, bytes) | 5 boolean (int32)
      3 table: int32 index, int32 count, count x (key, value)
      4 torch object: int32 index, string "V 1", string class, payload
          torch.<T>Tensor : int32 ndim, long sizes, long strides, long offset (1-based), storage
          torch.<T>Storage: long n, raw elements
          nn.<Module>     : a table with the module's fields
      an index that was written before stands for that earlier object.

Indices count the tables and torch objects in the order they are written,
starting at 1 -- Torch numbers them that way and the reference's reader
(thload.c:126-152, 262-301) relies on it.
"""
import struct

import numpy as np

TAG_NIL, TAG_NUMBER, TAG_STRING, TAG_TABLE, TAG_TORCH, TAG_BOOLEAN = 0, 1, 2, 3, 4, 5

_TENSOR_CLASS = {
    np.dtype(np.float32): "Float", np.dtype(np.float64): "Double", np.dtype(np.int64): "Long",
    np.dtype(np.int32): "Int", np.dtype(np.int16): "Short", np.dtype(np.uint8): "Byte", np.dtype(np.int8): "Char",
}
_CLASS_DTYPE = {v: k for k, v in _TENSOR_CLASS.items()}
_CLASS_DTYPE["Cuda"] = np.dtype(np.float32)


class Obj:
    """A torch object that is a table of fields: ``Obj("nn.Linear", weight=w, bias=b)``."""

    def __init__(self, cls, **fields):
        self.cls = cls
        self.fields = fields

    def __repr__(self):
        return "Obj(%s, %s)" % (self.cls, sorted(self.fields))


class Storage:
    """A bare storage (``torch.LongStorage`` for ``nn.View.size`` and the like)."""

    def __init__(self, data):
        self.data = np.ascontiguousarray(data)


class TensorView:
    """A tensor over a shared storage (Torch's flattened parameters look like this):
    element offset (0-based), sizes and strides in elements."""

    def __init__(self, storage, offset, size, stride):
        self.storage, self.offset, self.size, self.stride = storage, int(offset), list(size), list(stride)


class Writer:
    def __init__(self, fp, longsize=8):
        self.fp = fp
        self.long = "<q" if longsize == 8 else "<i"
        self.longsize = longsize
        self.index = {}          # id(python object) -> index
        self.next = 1
        self._keep = []          # keeps ids unique while writing
        self._private = {}       # id(array) -> the storage written for it

    def _int(self, v):
        self.fp.write(struct.pack("<i", v))

    def _long(self, v):
        self.fp.write(struct.pack(self.long, v))

    def _string(self, s):
        b = s.encode() if isinstance(s, str) else s
        self._int(len(b))
        self.fp.write(b)

    def _ref(self, obj):
        """Writes the index; True when the object was written before."""
        key = id(obj)
        if key in self.index:
            self._int(self.index[key])
            return True
        self._keep.append(obj)
        self.index[key] = self.next
        self._int(self.next)
        self.next += 1
        return False

    def _storage(self, arr, owner):
        flat = np.ascontiguousarray(arr).reshape(-1)
        self._int(TAG_TORCH)
        if self._ref(owner):
            return
        self._string("V 1")
        self._string("torch.%sStorage" % _TENSOR_CLASS[flat.dtype])
        self._long(flat.size)
        if flat.dtype == np.int64 and self.longsize == 4:
            flat = flat.astype(np.int32)
        self.fp.write(flat.tobytes())

    def _tensor(self, owner, dtype, size, stride, offset, storage):
        self._int(TAG_TORCH)
        if self._ref(owner):
            return
        self._string("V 1")
        self._string("torch.%sTensor" % _TENSOR_CLASS[np.dtype(dtype)])
        self._int(len(size))
        for v in size:
            self._long(v)
        for v in stride:
            self._long(v)
        self._long(offset + 1)
        if storage is None:
            self._int(TAG_NIL)
        else:
            self._storage(storage.data, storage)

    def write(self, obj):
        if obj is None:
            self._int(TAG_NIL)
        elif isinstance(obj, (bool, np.bool_)):
            self._int(TAG_BOOLEAN)
            self._int(1 if obj else 0)
        elif isinstance(obj, (int, float, np.integer, np.floating)):
            self._int(TAG_NUMBER)
            self.fp.write(struct.pack("<d", float(obj)))
        elif isinstance(obj, (str, bytes)):
            self._int(TAG_STRING)
            self._string(obj)
        elif isinstance(obj, (list, tuple)):
            self.write_table(obj, [(i + 1, v) for i, v in enumerate(obj)])
        elif isinstance(obj, dict):
            self.write_table(obj, list(obj.items()))
        elif isinstance(obj, np.ndarray):
            # a contiguous tensor over a storage of its own
            c = np.ascontiguousarray(obj)
            store = self._private.setdefault(id(obj), Storage(c))
            self._keep.append(obj)
            self._tensor(obj, c.dtype, c.shape, [st // c.itemsize for st in c.strides], 0, store if c.size else None)
        elif isinstance(obj, TensorView):
            self._tensor(obj, obj.storage.data.dtype, obj.size, obj.stride, obj.offset, obj.storage)
        elif isinstance(obj, Storage):
            self._storage(obj.data, obj)
        elif isinstance(obj, Obj):
            self._int(TAG_TORCH)
            if self._ref(obj):
                return
            self._string("V 1")
            self._string(obj.cls)
            self.write_table(obj.fields, list(obj.fields.items()))
        else:
            raise TypeError("cannot serialise %r" % type(obj))

    def write_table(self, owner, items):
        self._int(TAG_TABLE)
        if self._ref(owner):
            return
        self._int(len(items))
        for k, v in items:
            self.write(k)
            self.write(v)


def save(path, obj, longsize=8):
    with open(path, "wb") as fp:
        Writer(fp, longsize).write(obj)


# ---- reader (tests use it to check the writer against itself and to inspect files) ----

class Reader:
    def __init__(self, data, longsize=8):
        self.d = data
        self.p = 0
        self.longsize = longsize
        self.memo = {}

    def _unpack(self, fmt):
        n = struct.calcsize(fmt)
        v = struct.unpack_from(fmt, self.d, self.p)[0]
        self.p += n
        return v

    def _int(self):
        return self._unpack("<i")

    def _long(self):
        return self._unpack("<q" if self.longsize == 8 else "<i")

    def _string(self):
        n = self._int()
        s = self.d[self.p:self.p + n]
        self.p += n
        return s.decode()

    def read(self):
        tag = self._int()
        if tag == TAG_NIL:
            return None
        if tag == TAG_NUMBER:
            return self._unpack("<d")
        if tag == TAG_STRING:
            return self._string()
        if tag == TAG_BOOLEAN:
            return self._int() != 0
        if tag == TAG_TABLE:
            idx = self._int()
            if idx in self.memo:
                return self.memo[idx]
            t = self.memo[idx] = {}
            for _ in range(self._int()):
                k = self.read()
                t[k] = self.read()
            return t
        if tag == TAG_TORCH:
            idx = self._int()
            if idx in self.memo:
                return self.memo[idx]
            self._string()
            cls = self._string()
            if cls.startswith("torch.") and cls.endswith("Tensor"):
                dt = _CLASS_DTYPE[cls[6:-6]]
                nd = self._int()
                size = [self._long() for _ in range(nd)]
                stride = [self._long() for _ in range(nd)]
                off = self._long() - 1
                holder = self.memo[idx] = [None]
                st = self.read()
                if st is None:
                    arr = np.zeros(size, dt)
                else:
                    arr = np.lib.stride_tricks.as_strided(st.data[off:], size, [s * dt.itemsize for s in stride])
                holder[0] = arr
                self.memo[idx] = arr
                return arr
            if cls.startswith("torch.") and cls.endswith("Storage"):
                dt = _CLASS_DTYPE[cls[6:-7]]
                n = self._long()
                if dt == np.int64 and self.longsize == 4:
                    raw = np.frombuffer(self.d, np.int32, n, self.p).astype(np.int64)
                    self.p += 4 * n
                else:
                    raw = np.frombuffer(self.d, dt, n, self.p).copy()
                    self.p += dt.itemsize * n
                s = self.memo[idx] = Storage(raw)
                return s
            o = self.memo[idx] = Obj(cls)
            o.fields = self.read()
            return o
        raise ValueError("tag %d at byte %d" % (tag, self.p - 4))


def load(path, longsize=8):
    with open(path, "rb") as fp:
        return Reader(fp.read(), longsize).read()


# ---- layer lists (thnets_amd.netbuild) -> nn objects ----

def _f32(a):
    return np.ascontiguousarray(a, np.float32)


def module_of(spec, conv_as_4d=False, boolean_ceil=False):
    """One netbuild layer dict as the Torch7 nn object the reference's loaders read
    (field names: modules/*.c ``nnload_*``)."""
    kind = spec["type"]
    if kind == "conv":
        w = _f32(spec["weight"])
        co, ci, kh, kw = w.shape
        return Obj("nn.SpatialConvolution" if conv_as_4d else "nn.SpatialConvolutionMM",
                   padW=spec["padW"], padH=spec["padH"], dW=spec["dW"], dH=spec["dH"], kW=kw, kH=kh,
                   nInputPlane=ci, nOutputPlane=co, weight=w if conv_as_4d else w.reshape(co, ci * kh * kw),
                   bias=_f32(spec["bias"]))
    if kind == "linear":
        return Obj("nn.Linear", weight=_f32(spec["weight"]), bias=_f32(spec["bias"]))
    if kind == "threshold":
        if spec.get("alpha", 0.0):
            raise ValueError("a leaky threshold has no Torch7 nn.Threshold form")
        relu = spec.get("threshold", 0.0) == 0 and spec.get("val", 0.0) == 0
        return Obj("nn.ReLU" if relu else "nn.Threshold", threshold=spec.get("threshold", 0.0), val=spec.get("val", 0.0),
                   inplace=bool(spec.get("inplace", 1)))
    if kind in ("maxpool", "avgpool"):
        f = {k: spec.get(k, 0) for k in ("kW", "kH", "dW", "dH", "padW", "padH")}
        cm = spec.get("ceil_mode", 0)
        f["ceil_mode"] = bool(cm) if boolean_ceil else cm
        if kind == "avgpool":
            f["count_include_pad"] = spec.get("count_include_pad", 0)
            return Obj("nn.SpatialAveragePooling", **f)
        return Obj("nn.SpatialMaxPooling", **f)
    if kind == "view":
        return Obj("nn.View", numElements=spec["numElements"], size=Storage(np.array([spec["numElements"]], np.int64)))
    if kind == "softmax":
        return Obj("nn.SoftMax")
    if kind == "bn":
        return Obj("nn.SpatialBatchNormalization", running_mean=_f32(spec["running_mean"]), running_var=_f32(spec["running_var"]),
                   weight=_f32(spec["weight"]), bias=_f32(spec["bias"]), eps=spec.get("eps", 1e-5))
    if kind == "dropout":
        return Obj("nn.Dropout", p=spec.get("p", 0.5), inplace=bool(spec.get("inplace", 1)), v2=bool(spec.get("v2", 1)))
    if kind == "sequential":
        return sequential_of(spec["layers"], conv_as_4d, boolean_ceil)
    if kind == "concattable":
        branches = [b[0] if len(b) == 1 else {"type": "sequential", "layers": b} for b in spec["branches"]]
        return Obj("nn.ConcatTable", modules=[module_of(b, conv_as_4d, boolean_ceil) for b in branches])
    if kind == "fullconv":
        w = _f32(spec["weight"])
        ci, co, kh, kw = w.shape
        return Obj("nn.SpatialFullConvolution", padW=spec.get("padW", 0), padH=spec.get("padH", 0), dW=spec.get("dW", 1),
                   dH=spec.get("dH", 1), adjW=spec.get("adjW", 0), adjH=spec.get("adjH", 0), kW=kw, kH=kh, nInputPlane=ci,
                   nOutputPlane=co, weight=w, bias=None if spec.get("bias") is None else _f32(spec["bias"]))
    if kind == "caddtable":
        return Obj("nn.CAddTable", inplace=False)
    if kind == "csubtable":
        return Obj("nn.CSubTable")
    raise ValueError("unknown layer type %r" % kind)


def sequential_of(layers, conv_as_4d=False, boolean_ceil=False):
    """A ``maxunpool`` layer names its pooling by position in the same list; in the
    file it holds a reference to that very nn.SpatialMaxPooling object."""
    mods = []
    for s in layers:
        if s["type"] == "maxunpool":
            mods.append(Obj("nn.SpatialMaxUnpooling", pooling=mods[s["pooling"]]))
        else:
            mods.append(module_of(s, conv_as_4d, boolean_ceil))
    return Obj("nn.Sequential", modules=mods)


def save_model_dir(path, layers, mean=None, std=None, longsize=8, conv_as_4d=False, boolean_ceil=False):
    """Writes ``<path>/model.net`` and, when mean / std are given, ``<path>/stat.t7``:
    the directory layout ``THLoadNetwork`` reads (thapi.c:275, 303)."""
    import os
    os.makedirs(path, exist_ok=True)
    save(os.path.join(path, "model.net"), sequential_of(layers, conv_as_4d, boolean_ceil), longsize)
    if mean is not None:
        save(os.path.join(path, "stat.t7"), {"mean": _f32(mean), "std": _f32(std)}, longsize)
