"""``torch.save`` / ``torch.load`` of a ``torch.ClTensor`` in Torch7's binary file format.

What a ClTensor and a ClStorage write is the reference's (src/torch/generic/Tensor.cpp:1290-1345:
``int nDimension, long size[], long stride[], long storageOffset + 1``, then the storage as an
object; src/torch/generic/Storage.cpp:255-283: ``long size, float data[size]``, the device
buffer read back first).  The object framing around them is Torch7's ``File:writeObject``
(``torch/File.lua``, not part of the reference tree): ``int 4`` (a torch object), ``int index``
(1, 2, ... in order of first appearance; a repeated object writes only its index), and on first
appearance ``int len, "V 1"``, ``int len, class name``, then the object's own ``write``.  ``nil``
is ``int 0``.  Binary files are native-endian with 4-byte ints and 8-byte longs.  No Torch7 is
installed here to read a file back, so the framing is checked against hand-assembled bytes only.
"""
from __future__ import annotations

import struct
from typing import Optional, Sequence, Tuple

import numpy as np

TYPE_NIL, TYPE_TORCH = 0, 4
TENSOR_CLASSES = ("torch.ClTensor", "torch.FloatTensor")
STORAGE_CLASSES = ("torch.ClStorage", "torch.FloatStorage")


def _string(text: str) -> bytes:
    raw = text.encode("ascii")
    return struct.pack("=i", len(raw)) + raw


def encode_tensor(sizes: Sequence[int], strides: Sequence[int], offset0: int, storage: Optional[np.ndarray],
                  tensor_class: str = "torch.ClTensor", storage_class: str = "torch.ClStorage") -> bytes:
    """The bytes ``torch.save`` writes for one tensor over one storage (``offset0`` counts from 0).  The dimension
    count is the header's own field, written as it stands (src/torch/generic/Tensor.cpp:1296): an empty tensor,
    which has no storage, holds -1 there (src/lib/THClTensor.cpp:635); 0 means a point tensor, with its storage."""
    nd = len(sizes)
    assert len(strides) == nd
    nd_field = -1 if (nd == 0 and storage is None) else nd
    out = [struct.pack("=ii", TYPE_TORCH, 1), _string("V 1"), _string(tensor_class),
           struct.pack("=i", nd_field), struct.pack("=%dq" % nd, *sizes), struct.pack("=%dq" % nd, *strides),
           struct.pack("=q", offset0 + 1)]
    if storage is None:
        out.append(struct.pack("=i", TYPE_NIL))
    else:
        data = np.ascontiguousarray(storage, dtype=np.float32).reshape(-1)
        out += [struct.pack("=ii", TYPE_TORCH, 2), _string("V 1"), _string(storage_class),
                struct.pack("=q", data.size), data.tobytes()]
    return b"".join(out)


class _Reader:
    def __init__(self, raw: bytes):
        self.raw, self.pos = raw, 0

    def take(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.raw):
            raise ValueError("file ends inside a field")
        v = struct.unpack_from(fmt, self.raw, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        (n,) = self.take("=i")
        if n < 0 or self.pos + n > len(self.raw):
            raise ValueError("bad string length")
        s = self.raw[self.pos:self.pos + n].decode("ascii")
        self.pos += n
        return s

    def header(self, classes: Tuple[str, ...], index: int) -> str:
        kind, idx = self.take("=ii")
        if kind != TYPE_TORCH or idx != index:
            raise ValueError(f"expected torch object #{index}, found type {kind} index {idx}")
        version, name = self.string(), self.string()
        if not version.startswith("V "):
            raise ValueError(f"unsupported version tag {version!r}")
        if name not in classes:
            raise ValueError(f"cannot read a {name}")
        return name


def decode_tensor(raw: bytes):
    """Inverse of :func:`encode_tensor`: ``(sizes, strides, offset0, storage or None, tensor_class, storage_class)``."""
    r = _Reader(raw)
    tclass = r.header(TENSOR_CLASSES, 1)
    (nd,) = r.take("=i")
    if nd == -1:
        nd = 0          # the reference writes its header field as is, and its empty header holds -1
    if nd < 0 or nd > 64:
        raise ValueError("bad dimension count")
    sizes = list(r.take("=%dq" % nd)) if nd else []
    strides = list(r.take("=%dq" % nd)) if nd else []
    (offset1,) = r.take("=q")
    (kind,) = r.take("=i")
    if kind == TYPE_NIL:
        return sizes, strides, offset1 - 1, None, tclass, None
    r.pos -= 4
    sclass = r.header(STORAGE_CLASSES, 2)
    (n,) = r.take("=q")
    if n < 0 or r.pos + 4 * n > len(raw):
        raise ValueError("storage is longer than the file")
    storage = np.frombuffer(raw, dtype=np.float32, count=n, offset=r.pos).copy()
    return sizes, strides, offset1 - 1, storage, tclass, sclass


def save(path: str, tensor) -> None:
    """``torch.save(path, clTensor)``: header plus the whole storage the tensor views."""
    from .tensor import _call
    nd = tensor.nDimension()
    if nd < 0 or (nd > 0 and tensor.nElement() == 0):          # empty; a point tensor has 0 dimensions and a storage
        raw = encode_tensor([], [], 0, None)
    else:
        st = _call("THClTensor_storage", tensor._h)
        n = int(_call("THClStorage_size", st))
        whole = tensor.strided([n], [1], 1).float() if n else np.zeros(0, dtype=np.float32)
        raw = encode_tensor(list(tensor.size()), list(tensor.stride()), tensor.storageOffset() - 1, whole)
    with open(path, "wb") as f:
        f.write(raw)


def load(path: str):
    """``torch.load(path)`` of a file holding one ClTensor (or FloatTensor): a ClTensor over a fresh storage."""
    from .tensor import ClTensor
    with open(path, "rb") as f:
        sizes, strides, offset0, storage, _, _ = decode_tensor(f.read())
    if storage is None:
        return ClTensor()
    if not sizes:
        # no dimensions but a storage: a point tensor, whose one value sits at the offset.  It is
        # rebuilt as the sum of that one element (exact: one fp64 addend, one rounding back).
        if not 0 <= offset0 < storage.size:
            return ClTensor()
        point = ClTensor()
        point.sum(ClTensor(storage[offset0:offset0 + 1]))
        return point
    need = offset0 + sum((s - 1) * t for s, t in zip(sizes, strides)) + 1
    if any(s <= 0 for s in sizes) or any(t < 0 for t in strides) or offset0 < 0 or need > storage.size:
        raise ValueError("tensor header points outside its storage")
    return ClTensor(storage).strided(sizes, strides, offset0 + 1)
